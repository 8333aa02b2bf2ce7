// Split-K decode attention over a quantized KV cache for gfx950 (wave64, MFMA).
//
// One workgroup (4 waves) owns one (kv head, key split, work item = the (row, head) columns of a slot
// or a part of them).  Each wave walks its own 32-key tiles of the split with a private online softmax
// and no workgroup barrier in the loop; the four waves merge in LDS at the end and write one
// unnormalised partial per (row, head, split).  A second kernel merges the splits.
//
// Two split kernels live here.
//
// decode_q8_kernel (q8_0, the shipped path; described where it is defined): the rows of a tile go
// from the cache to LDS as they lie (global_load_lds), and the MFMA operands are made where they are
// read.  Work items carry up to 8 columns (the two f16 halves of Q share one MFMA) or 9 to 16 (two MFMAs).
//
// decode_staged_kernel (q4_0, and q8_0 with fp32-class weights): the first kernel of this build.
// Memory pipeline: a tile's K (or V) rows are 32 x 272 contiguous bytes.  A
// lane fetches "units" of 68 bytes = two whole 34-byte blocks of one key, with
// dword-aligned 128-bit loads; a wave's load instruction covers a
// contiguous 4,352-byte span.  Two tiles (K and V each) are kept in flight per
// wave in registers.  On arrival a unit is realigned (the even block's payload
// sits 2 bytes into a dword) and written to a padded, aligned LDS tile
// [32 keys][288 B]; block scales go to a transposed f16 table [8 blocks][32 keys].
// K and V of a tile use the same LDS tile one after the other.
//
// Arithmetic of both (all MFMAs are v_mfma_f32_16x16x32_f16):
//   S^T[key][n]  = K[key][:] . Q^T[:][n]      A = K bytes as f16, B = Q (hi + lo f16)
//   O^T[d][n]   += V^T[d][key] . P'[key][n]   A = V bytes as f16 (LDS transpose read),
//                                              B = P' = p * scale_of_block(key, d/32)
// n runs over (query row, head) pairs, at most 16 per workgroup: a slot with more (3-4 MTP
// rows x 6-8 heads) is cut by heads into work items.  The C layout of S^T (row = 4*(lane/16)+i, col = lane%16)
// is exactly the B layout the PV product needs, so probabilities never leave
// their lane, and every per-column scalar (max, sum, rescale) lives in lane%16.
//
// Exactness:
//   - int8 -> f16 without rounding: byte b^0x80 = b+128 placed in the low byte of
//     an f16 is the subnormal (b+128)*2^-24; the offset of 128 is removed exactly (a packed f16
//     subtract in the staged kernel, a bias term in the other), and MFMA multiplies subnormals exactly.
//   - one q8 block (32 values) is one MFMA contraction, so the f16 block scale
//     multiplies an exact integer dot product in fp32 (as the CPU definition's
//     d * q does, crates/hipml-core/src/ops.rs:486-515 of the reference).
//   - Q is split into hi + lo f16 halves (~22 bits); the fp32-class variant splits P' as well.

#include "common.h"

#include <atomic>
#include <mutex>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>
#include <type_traits>

namespace hipml {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef int int2v __attribute__((ext_vector_type(2)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4a4 __attribute__((ext_vector_type(4), aligned(4)));

// ---- phase stamps (instrumented builds only: -DHIPML_DECODE_STAMPS, see hipml_amd/decode_phases.py) ------
// Wave 0 of every workgroup of decode_q8_kernel keeps the 100 MHz counter's value at up to kStampsPerWg points
// in scalar registers and writes them out when the kernel is done with its own memory traffic (a store in
// between would count among the requests the kernel's explicit waits are sized for).  Off, the macros are empty.
constexpr int kStampsPerWg = 12, kStampWgs = 4096;
#ifdef HIPML_DECODE_STAMPS
static __device__ unsigned long long decode_stamps[kStampWgs * kStampsPerWg];
struct Stamps { unsigned long long t[kStampsPerWg]; };
#define HIPML_STAMPS_DECL Stamps stamps_ = {}
#define HIPML_STAMP(st, i) ((st).t[i] = __builtin_amdgcn_s_memrealtime())
#define HIPML_STAMPS_ARG , Stamps &stamps_
#define HIPML_STAMPS_PASS , stamps_
__device__ __forceinline__ void stamps_out(const Stamps &st)
{
    const unsigned wg = blockIdx.x + gridDim.x * blockIdx.y;
    if (threadIdx.x == 0 && wg < kStampWgs)
        for (int i = 0; i < kStampsPerWg; i++)
            decode_stamps[wg * kStampsPerWg + i] = st.t[i];
}
int decode_read_stamps(unsigned long long *host, size_t n)
{
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(decode_stamps), (n < (size_t)kStampWgs * kStampsPerWg ? n : (size_t)kStampWgs * kStampsPerWg) * sizeof(unsigned long long));
}
#else
#define HIPML_STAMPS_DECL
#define HIPML_STAMP(st, i) ((void)0)
#define HIPML_STAMPS_ARG
#define HIPML_STAMPS_PASS
#endif

constexpr int kMaxItems = 4 * kMaxSlots;               // work items of one launch (see DecodeArgs)
constexpr int kTileKeys = 32;                         // keys per wave tile
constexpr int kLdsRow = 288;                          // 256 payload bytes + 32 pad (bank spread)
constexpr int kTileBytes = kTileKeys * kLdsRow;       // 9216: payload tile (K, then V)
constexpr int kScaleBytes = 8 * kTileKeys * 2;        // 512: f16 [8 blocks][32 keys]
constexpr int kWaveLds = kTileBytes + 2 * kScaleBytes; // 10240
constexpr int kWaves = 4;            // waves per workgroup
constexpr int kThreads = 64 * kWaves;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kTwo24 = 16777216.0f;
// Opaque use-and-redefine of a register: the value must exist here, in a VGPR.
#define PIN(x) asm volatile("" : "+v"(x))

constexpr int kQLds = 16384 + 2048; // per column tile: Q operands (hi, lo) + bias table
constexpr int decode_lds_bytes(int nt) { return nt * kQLds + kWaves * kWaveLds; }

struct DecodeArgs {
    const float *q;
    const uint8_t *k;
    const uint8_t *v;
    float *part_acc;
    float *part_ml;
    const int32_t *pos;
    int n_kv, group, stride, splits;
    int items;     // work items (grid.y of a plain launch)
    // item 0 once more, as plain scalars: a launch with a single item (one sequence, one query row)
    // then needs no table lookup, which is a vector load from the kernel-argument segment and a
    // memory round trip before the first Q and K/V requests can be addressed
    int i0_row0, i0_cols, i0_slot, i0_head0, i0_nhead;
    int workers;   // > 0: worker launch, workgroups per KV head (see decode_body)
    int stream_once; // the launch has one work item, so the cache rows are read once (non-temporal loads);
                     // the kernel decides the same per item for launches with several
    float scale_log2; // scale * log2(e) * 2^24
    size_t kv_slot_bytes, acc_slot, ml_slot, q_slot;
    // merge > 0: the workgroups of a plain launch merge their partials themselves (decode_merge_tail),
    // in groups of `merge` splits first; `tickets` are that launch's arrival counters
    float *out;
    const float *gate;
    unsigned int *tickets;
    int merge;
    // Work items (grid.y).  A slot whose rows x heads fit the columns of one workgroup (16; the raw-row
    // kernel runs items of up to 8 columns through its narrow body and wider ones through its wide
    // one) is one item; a wider one (2-4 MTP rows x 6 heads) is cut by heads into
    // items that stream the same cache rows: their workgroups are gridDim.x apart in launch order, a
    // multiple of the 8 XCDs here, so the later readers find the rows in the first one's L2.
    uint16_t row0[kMaxItems];  // first query row of the item's slot
    uint8_t cols[kMaxItems];   // query rows of the slot (1..kMaxCols)
    uint8_t kvslot[kMaxItems]; // slot index, for the cache base
    uint8_t head0[kMaxItems];  // first head (within the GQA group) of the item
    uint8_t nhead[kMaxItems];  // heads of the item
};

// What a workgroup needs before it can ask for its first rows.  decode_q8_kernel takes these as leading scalar
// kernel arguments, which arrive in registers with the wave (the argument structure behind them is fetched from
// memory: a round trip of ~0.4 us before "work item found" while everything sat there); the staged kernels fill
// the same view from the structure.
struct Front {
    const uint8_t *k, *v; // (a launch with one item: already at that item's slot)
    const float *q;
    const int32_t *pos;
    int stride, splits, workers, items;
    int i0_row0, i0_cols, i0_slot, i0_head0, i0_nhead;
    int group, n_kv, stream_once;
    uint32_t q_slot;
    uint32_t karg_at; // where the argument structure lies in the kernel-argument segment
};
__device__ __forceinline__ Front front_of(const DecodeArgs &a)
{
    Front f;
    f.k = a.k;
    f.v = a.v;
    f.q = a.q;
    f.pos = a.pos;
    f.stride = a.stride;
    f.splits = a.splits;
    f.workers = a.workers;
    f.items = a.items;
    f.i0_row0 = a.i0_row0;
    f.i0_cols = a.i0_cols;
    f.i0_slot = a.i0_slot;
    f.i0_head0 = a.i0_head0;
    f.i0_nhead = a.i0_nhead;
    f.group = a.group;
    f.n_kv = a.n_kv;
    f.stream_once = a.stream_once;
    f.q_slot = (uint32_t)a.q_slot;
    f.karg_at = 0;
    return f;
}
// The leading arguments of decode_q8_kernel, packed on the host (pack_front) and taken apart here.
struct FrontWords { uint32_t wi, item0, geom; };
__device__ __forceinline__ Front front_of(const uint8_t *k, const uint8_t *v, const float *q, const int32_t *pos, int stride,
                                          int splits, uint32_t wi, uint32_t item0, uint32_t geom, uint32_t q_slot,
                                          uint32_t karg_at)
{
    Front f;
    f.k = k;
    f.v = v;
    f.q = q;
    f.pos = pos;
    f.stride = stride;
    f.splits = splits;
    f.workers = (int)(wi & 0xffffu);
    f.items = (int)(wi >> 16);
    f.i0_row0 = (int)(item0 & 0x3ffu);
    f.i0_cols = (int)(item0 >> 10 & 7u);
    f.i0_head0 = (int)(item0 >> 13 & 7u);
    f.i0_nhead = (int)(item0 >> 16 & 15u);
    f.i0_slot = (int)(item0 >> 20 & 0xffu);
    f.group = (int)(geom & 15u);
    f.n_kv = (int)(geom >> 4 & 0xffffu);
    f.stream_once = (int)(geom >> 20 & 1u);
    f.q_slot = q_slot;
    f.karg_at = karg_at;
    return f;
}

// 68 bytes of a key row starting at a block-pair boundary: [s0 | 32 x i8 | s1 | 32 x i8].
struct Unit {
    uint4v a, b; // dwords 0..7:  s0 and the first 30 bytes of the even block
    uint32_t m;  // dword 8:      last 2 bytes of the even block, s1
    uint4v c, d; // dwords 9..16: the odd block's 32 bytes (dword aligned)
};

// Plain (cached) loads: the five loads of a unit and its neighbours' share 128-byte lines, and
// a non-temporal hint makes every one of them fetch the line again (measured: 3.3 vs 5.6 TB/s).
__device__ __forceinline__ void load_unit(Unit &u, const uint8_t *p)
{
    u.a = *reinterpret_cast<const uint4a4 *>(p);
    u.b = *reinterpret_cast<const uint4a4 *>(p + 16);
    u.m = *reinterpret_cast<const uint32_t *>(p + 32);
    u.c = *reinterpret_cast<const uint4a4 *>(p + 36);
    u.d = *reinterpret_cast<const uint4a4 *>(p + 52);
}

// Realign one unit and store it: payloads of blocks (2*pr, 2*pr+1) of tile row r to the padded
// tile, their scales to the transposed table.
// A row past the live length (`live` false) gets zero scales: its bytes are whatever the cache
// holds there, and a non-finite scale would turn its zero weight into NaN.
__device__ __forceinline__ void store_unit(const Unit &u, uint8_t *tile, uint8_t *scales, int r,
                                           int pr, bool live)
{
    uint4v e0, e1;
    e0[0] = __builtin_amdgcn_alignbit(u.a[1], u.a[0], 16);
    e0[1] = __builtin_amdgcn_alignbit(u.a[2], u.a[1], 16);
    e0[2] = __builtin_amdgcn_alignbit(u.a[3], u.a[2], 16);
    e0[3] = __builtin_amdgcn_alignbit(u.b[0], u.a[3], 16);
    e1[0] = __builtin_amdgcn_alignbit(u.b[1], u.b[0], 16);
    e1[1] = __builtin_amdgcn_alignbit(u.b[2], u.b[1], 16);
    e1[2] = __builtin_amdgcn_alignbit(u.b[3], u.b[2], 16);
    e1[3] = __builtin_amdgcn_alignbit(u.m, u.b[3], 16);
    uint4v *dst = reinterpret_cast<uint4v *>(tile + r * kLdsRow + pr * 64);
    dst[0] = e0;
    dst[1] = e1;
    dst[2] = u.c;
    dst[3] = u.d;
    uint16_t *sc = reinterpret_cast<uint16_t *>(scales) + (2 * pr) * kTileKeys + r;
    sc[0] = live ? (uint16_t)(u.a[0] & 0xffffu) : (uint16_t)0;
    sc[kTileKeys] = live ? (uint16_t)(u.m >> 16) : (uint16_t)0;
}

// q4_0: a unit is two 18-byte blocks of one key, 36 bytes at a dword boundary:
// [s0 | 16 bytes | s1 | 16 bytes]; byte j of a block holds element j in its low and element j+16
// in its high nibble (crates/hipml-core/src/kv.rs:201-218).
struct Unit4 {
    uint4v a;   // dwords 0..3: s0 and the first 14 bytes of the even block
    uint32_t m; // dword 4:     last 2 bytes of the even block, s1
    uint4v b;   // dwords 5..8: the odd block's 16 bytes (dword aligned)
};

__device__ __forceinline__ void load_unit(Unit4 &u, const uint8_t *p)
{
    u.a = *reinterpret_cast<const uint4a4 *>(p);
    u.m = *reinterpret_cast<const uint32_t *>(p + 16);
    u.b = *reinterpret_cast<const uint4a4 *>(p + 20);
}

// Nibbles widened to one byte per element (values 0..15), element order, so the tile has the
// q8_0 tile's shape and everything after staging is shared; the offset to remove is 8, not 128.
__device__ __forceinline__ void store_unit(const Unit4 &u, uint8_t *tile, uint8_t *scales, int r,
                                           int pr, bool live)
{
    uint4v e0;
    e0[0] = __builtin_amdgcn_alignbit(u.a[1], u.a[0], 16);
    e0[1] = __builtin_amdgcn_alignbit(u.a[2], u.a[1], 16);
    e0[2] = __builtin_amdgcn_alignbit(u.a[3], u.a[2], 16);
    e0[3] = __builtin_amdgcn_alignbit(u.m, u.a[3], 16);
    const uint4v mask = {0x0f0f0f0fu, 0x0f0f0f0fu, 0x0f0f0f0fu, 0x0f0f0f0fu};
    uint4v *dst = reinterpret_cast<uint4v *>(tile + r * kLdsRow + pr * 64);
    dst[0] = e0 & mask;
    dst[1] = (e0 >> 4) & mask;
    dst[2] = u.b & mask;
    dst[3] = (u.b >> 4) & mask;
    uint16_t *sc = reinterpret_cast<uint16_t *>(scales) + (2 * pr) * kTileKeys + r;
    sc[0] = live ? (uint16_t)(u.a[0] & 0xffffu) : (uint16_t)0;
    sc[kTileKeys] = live ? (uint16_t)(u.m >> 16) : (uint16_t)0;
}

template <bool Q4> struct UnitOf { typedef Unit type; };
template <> struct UnitOf<true> { typedef Unit4 type; };

// 8 int8 b -> 8 f16 holding (b + 128) * 2^-24 exactly (byte b^0x80 in the low byte of a
// subnormal f16).  The +128 is taken out again on the B side: sum_k (u_k - 128) x_k =
// sum_k u_k x_k - 128 sum_k x_k.  For the scores x = Q is fixed, so the second term is a table
// the block's MFMA starts from; for PV it is a second MFMA whose A operand is the constant
// -128 * 2^-24.
// (q4_0 tiles already hold unsigned bytes 0..15: no sign flip, and the offset is 8.)
template <bool Q4>
__device__ __forceinline__ half8 bytes_to_f16_biased(int2v w)
{
    const uint32_t x0 = Q4 ? (uint32_t)w[0] : (uint32_t)w[0] ^ 0x80808080u;
    const uint32_t x1 = Q4 ? (uint32_t)w[1] : (uint32_t)w[1] ^ 0x80808080u;
    uint4v r;
    r[0] = __builtin_amdgcn_perm(0u, x0, 0x0c010c00u);
    r[1] = __builtin_amdgcn_perm(0u, x0, 0x0c030c02u);
    r[2] = __builtin_amdgcn_perm(0u, x1, 0x0c010c00u);
    r[3] = __builtin_amdgcn_perm(0u, x1, 0x0c030c02u);
    return __builtin_bit_cast(half8, r);
}

// max / sum over the four lanes {l, l^16, l^32, l^48} without LDS (row-swap instructions,
// written as asm: the compiler's builtins for them return the first result twice)
template <bool MAX>
__device__ __forceinline__ float quad_rows(float v)
{
    float a = v, b = v;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    v = MAX ? fmaxf(a, b) : a + b;
    a = v;
    b = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return MAX ? fmaxf(a, b) : a + b;
}

// The work of one workgroup: which KV head, work item and key split it serves.
struct Work {
    int kvh, split, nsp, item;              // KV head, split index, splits of this item that have workers, item index
    int slot, row0, ncols, group, head0;    // the item: cache slot, first query row, rows, heads, first head
    int hbase, nvalid;                      // first head overall, (row, head) columns of the item
};

// Returns false when this workgroup has nothing to do (uniform over the workgroup).
__device__ __forceinline__ bool find_work(const DecodeArgs &a, const Front &f, int lane, Work &wk)
{
    // ---- which (kv head, item, split) this workgroup is ---------------------------------------
    // Plain launches: grid (n_kv * splits, items), every split of every item gets tiles.
    // Worker launches (batches, f.workers > 0): grid (n_kv * workers).  The hardware starts the
    // workgroups of a launch in windows of as many as fit the chip (512 here) and opens the next
    // window only when the whole previous one has finished, so a workgroup with little or nothing to
    // do still holds its place for as long as the longest one of its window.  A batch has items of
    // very different depth: its launch is therefore exactly one window of workers, and each worker
    // derives its (item, split) from the live lengths in device memory: item i gets
    // nsp_i = clamp(ceil(tiles_i / T), 1, splits) consecutive workers, T the smallest number of
    // tiles per worker for which these add up to no more than `workers` (the launcher keeps
    // items <= workers), i.e. no worker has more than T tiles.
    int kvh, split, item, nsp;
    // The scalar arguments span two 64-byte lines of the kernel-argument segment, both cold when a
    // workgroup starts.  Left alone the compiler fetches `workers` (second line) here and the first
    // line only where the pointers are first used: two memory round trips one after the other.  A
    // condition over one field of each line asks for both at once (`stride` is positive, checked by
    // the launcher).
    const bool worker_launch = (f.workers > 0) & (f.stride > 0);
    if (worker_launch) {
        kvh = blockIdx.x / f.workers;
        const int w = blockIdx.x - kvh * f.workers;
        // lane i looks at item i (the launcher uses this mode for at most 64 items); item tables
        // are read through the kernel-argument pointer: a lane-indexed read of the by-value
        // argument struct would make the compiler copy its arrays to scratch
        typedef const __attribute__((address_space(4))) uint8_t *KargBytes;
        typedef const __attribute__((address_space(4))) uint16_t *KargHalves;
        const KargBytes ka = (KargBytes)__builtin_amdgcn_kernarg_segment_ptr();
        const KargHalves t_row0 = (KargHalves)(ka + f.karg_at + offsetof(DecodeArgs, row0));
        const KargBytes t_cols = ka + f.karg_at + offsetof(DecodeArgs, cols);
        int tiles = 0;
        if (lane < f.items) {
            const int r0 = t_row0[lane], nc = t_cols[lane];
            int sm = 0;
            for (int c = 0; c < nc; c++) {
                int v = f.pos[(size_t)(r0 + c) * 2 + 1];
                v = v < 0 ? 0 : (v > f.stride ? f.stride : v);
                sm = v > sm ? v : sm;
            }
            tiles = (sm + kTileKeys - 1) / kTileKeys;
        }
        // the smallest number T of tiles per worker for which the items' shares ceil(tiles / T)
        // (at least one worker each, at most `splits`) fit the workers there are: no worker then has
        // more than T tiles, whatever the mix of depths (shares proportional to the tiles and rounded
        // down left some items with half as many workers again as they needed)
        int tmax = tiles, total = tiles;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const int o = __shfl_xor(tmax, off);
            tmax = o > tmax ? o : tmax;
            total += __shfl_xor(total, off);
        }
        auto share_at = [&](int t) {
            int sh = 0;
            if (lane < f.items) {
                // ceil(tiles / t) through a float quotient (tiles < 2^24: exact or one too many at a
                // multiple, corrected below); every wave computes the same values
                sh = (int)((float)tiles / (float)t);
                sh += sh * t < tiles ? 1 : 0;
                sh -= (sh - 1) * t >= tiles && sh > 0 ? 1 : 0;
                sh = sh < 1 ? 1 : (sh < f.splits ? sh : f.splits);
            }
            return sh;
        };
        // T lies between total / workers and total / (workers - items) (each share is below
        // tiles / T + 1), so the search is a few steps
        const int spare = f.workers - f.items;
        int lo = (total + f.workers - 1) / f.workers;
        lo = lo < 1 ? 1 : lo;
        int hi = spare > 0 ? (total + spare - 1) / spare : (tmax > 1 ? tmax : 1);
        hi = hi < lo ? lo : hi;
        while (lo < hi) { // uniform over the wave
            const int mid = (lo + hi) >> 1;
            int need = share_at(mid);
#pragma unroll
            for (int off = 32; off > 0; off >>= 1)
                need += __shfl_xor(need, off);
            if (need <= f.workers)
                hi = mid;
            else
                lo = mid + 1;
        }
        const int share = share_at(lo);
        int end = share; // inclusive prefix sum over lanes
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int up = __shfl_up(end, off);
            end += lane >= off ? up : 0;
        }
        const unsigned long long hit = __ballot(lane < f.items && w >= end - share && w < end);
        if (hit == 0)
            return false; // more workers than the shares add up to (uniform over the workgroup)
        item = __builtin_ctzll(hit);
        nsp = __shfl(share, item);
        split = w - (__shfl(end, item) - nsp);
        item = __builtin_amdgcn_readfirstlane(item);
        nsp = __builtin_amdgcn_readfirstlane(nsp);
        split = __builtin_amdgcn_readfirstlane(split);
    } else {
        kvh = blockIdx.x / f.splits;
        split = blockIdx.x - kvh * f.splits;
        item = blockIdx.y;
        nsp = f.splits;
    }
    // The item tables are byte arrays read with vector loads, and the item is the same for every lane.
    // Taking the values through readfirstlane puts them in scalar registers and, more to the point,
    // makes the wave wait for them here, while nothing else is outstanding: the (conditional) Q loads
    // below come later in the same in-order queue, so a first use behind them would wait for the Q
    // rows as well, and the first tile could only be requested once those had arrived.
    int slot, row0, ncols, group, head0; // group = heads of this item: columns are (row, head) pairs over them
    if (f.items == 1) {
        slot = f.i0_slot;
        row0 = f.i0_row0;
        ncols = f.i0_cols;
        group = f.i0_nhead;
        head0 = f.i0_head0;
    } else {
        slot = __builtin_amdgcn_readfirstlane((int)a.kvslot[item]);
        row0 = __builtin_amdgcn_readfirstlane((int)a.row0[item]);
        ncols = __builtin_amdgcn_readfirstlane((int)a.cols[item]);
        group = __builtin_amdgcn_readfirstlane((int)a.nhead[item]);
        head0 = __builtin_amdgcn_readfirstlane((int)a.head0[item]);
    }
    const int hbase = kvh * f.group + head0;
    const int nvalid = ncols * group;
    if (f.workers > 0 && split == 0 && nsp < f.splits) {
        // the splits of this item that no worker takes: empty partials, which the merge skips
        const int empty = f.splits - nsp;
        for (int e = threadIdx.x; e < nvalid * empty; e += (int)blockDim.x) {
            const int n = e / empty, sp = nsp + (e - n * empty);
            const int col = n / group;
            const int head = hbase + (n - col * group);
            float *pm = a.part_ml + (size_t)(row0 + col) * a.ml_slot + ((size_t)head * f.splits + sp) * 2;
            pm[0] = -INFINITY;
            pm[1] = 0.0f;
        }
    }

    wk.kvh = kvh;
    wk.split = split;
    wk.nsp = nsp;
    wk.item = item;
    wk.slot = slot;
    wk.row0 = row0;
    wk.ncols = ncols;
    wk.group = group;
    wk.head0 = head0;
    wk.hbase = hbase;
    wk.nvalid = nvalid;
    return true;
}

template <int NT, bool Q4, bool PLO>
__device__ __forceinline__ void decode_body(const DecodeArgs &a)
{
    typedef typename UnitOf<Q4>::type Unit;
    constexpr int kRowBytes = Q4 ? hipml::kRowBytesQ4 : hipml::kRowBytes;
    constexpr int kUnitBytes = Q4 ? 36 : 68;
    constexpr float kOffset = Q4 ? 8.0f : 128.0f; // what a staged byte carries on top of the value
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_all[];
    uint8_t *Qs = lds_all;                       // [NT][hi,lo][8 blocks][64 lanes] half8
    uint8_t *CBs = lds_all + NT * 16384;         // [NT][8 blocks][16 columns] float4 (one value x4)
    uint8_t *wave_base = lds_all + NT * kQLds;   // per-wave tile + scale tables

    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int lm = lane & 15; // MFMA row/col within the 16-tile
    const int lg = lane >> 4; // k-group
    const Front f = front_of(a);
    Work wk;
    if (!find_work(a, f, lane, wk))
        return;
    const int kvh = wk.kvh, split = wk.split, nsp = wk.nsp, slot = wk.slot, row0 = wk.row0, ncols = wk.ncols,
              group = wk.group, hbase = wk.hbase, nvalid = wk.nvalid;

    uint8_t *tile_lds = wave_base + wave * kWaveLds;
    uint8_t *sK = tile_lds + kTileBytes;
    uint8_t *sV = sK + kScaleBytes;

    const uint8_t *kbase = f.k + (size_t)slot * a.kv_slot_bytes + (size_t)kvh * f.stride * kRowBytes;
    const uint8_t *vbase = f.v + (size_t)slot * a.kv_slot_bytes + (size_t)kvh * f.stride * kRowBytes;

    // ---- key tiles of this wave ---------------------------------------------------------------
    // The 32-key tiles of a KV head are dealt round-robin: tile g belongs to split (g / kWaves)
    // % nsp, wave g % kWaves, so wave `wave` of split `split` owns tiles
    // (t * nsp + split) * kWaves + wave, t = 0, 1, ...  In a plain launch the addresses depend on
    // the launch only, not on the live length, which lives in device memory: the first tile is
    // requested before that length has been read (a tile past the live rows costs one load of rows
    // inside the cache's stride and is masked out), and neighbouring workgroups stream neighbouring rows.
    auto tile_key0 = [&](int t) { return ((t * nsp + split) * kWaves + wave) * kTileKeys; };

    // ---- staging registers: one tile in flight, 2 K units + 2 V units per lane -----------------
    Unit Kst[2], Vst[2];
    // unit j of a tile: u = lane + 64*j -> tile row u/4, block pair u%4
    const int ur0 = lane >> 2, ur1 = 16 + (lane >> 2), upr = lane & 3;
    const int last_row = f.stride - 1;
    auto issue = [&](Unit (&dst)[2], const uint8_t *base, int t) {
        const int key0 = tile_key0(t);
        int ka = key0 + ur0, kb = key0 + ur1;
        ka = ka < last_row ? ka : last_row; // never leave the cache; rows past the live length are
        kb = kb < last_row ? kb : last_row; // neutralised when they are staged
        load_unit(dst[0], base + (size_t)ka * kRowBytes + upr * kUnitBytes);
        load_unit(dst[1], base + (size_t)kb * kRowBytes + upr * kUnitBytes);
    };

    // ---- Q rows first: their addresses need nothing from device memory.  Entry (nt, c, l) of the
    // LDS operand table = Q[col n = nt*16 + l%16][c*32 + (l/16)*8 .. +8]; a thread owns entries tid + kThreads*k.
    constexpr int kQEntries = NT * 8 * 64 / kThreads;
    float4v qf[kQEntries][2];
#pragma unroll
    for (int k = 0; k < kQEntries; k++) {
        const int e = threadIdx.x + kThreads * k;
        const int l = e & 63, c = (e >> 6) & 7, nt = e >> 9;
        const int n = nt * 16 + (l & 15);
        qf[k][0] = (float4v){0, 0, 0, 0};
        qf[k][1] = (float4v){0, 0, 0, 0};
        if (n < nvalid) {
            const int col = n / group;
            const int head = n - col * group;
            const float *qp = f.q + (size_t)(row0 + col) * f.q_slot +
                              (size_t)(hbase + head) * kHeadDim + c * 32 + (l >> 4) * 8;
            qf[k][0] = *reinterpret_cast<const float4v *>(qp);
            qf[k][1] = *reinterpret_cast<const float4v *>(qp + 4);
        }
    }

    // ... and right behind them the first tile: loads return in order, so the few Q rows are not
    // queued behind 17 KB of K/V, and the tile is on its way before the live length is known
    issue(Kst, kbase, 0);
    issue(Vst, vbase, 0);

    // live lengths of this slot's rows
    int seqc[kMaxCols];
    int seq_max = 0;
#pragma unroll
    for (int c = 0; c < kMaxCols; c++) {
        int s = c < ncols ? f.pos[(size_t)(row0 + c) * 2 + 1] : 0;
        s = s < 0 ? 0 : (s > f.stride ? f.stride : s);
        seqc[c] = s;
        seq_max = s > seq_max ? s : seq_max;
    }
    const int hi = seq_max; // keys at or past it are masked
    if (split * kWaves * kTileKeys >= hi) {
        // not one live tile for any wave of this workgroup (a shallow slot of a batch, or more
        // splits than tiles): leave an empty partial and go, the merge skips it
        if ((int)threadIdx.x < nvalid) {
            const int col = threadIdx.x / group;
            const int head = hbase + (threadIdx.x - col * group);
            float *pm = a.part_ml + (size_t)(row0 + col) * a.ml_slot + ((size_t)head * f.splits + split) * 2;
            pm[0] = -INFINITY;
            pm[1] = 0.0f;
        }
        return; // uniform over the workgroup
    }
    const int first_key = tile_key0(0), step_keys = nsp * kWaves * kTileKeys;
    const int ntile = first_key < hi ? (hi - first_key + step_keys - 1) / step_keys : 0;

    // ---- Q operands to LDS as hi + lo f16 ------------------------------------------------------
#pragma unroll
    for (int k = 0; k < kQEntries; k++) {
        const int e = threadIdx.x + kThreads * k;
        half8 h8, l8;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float x = j < 4 ? qf[k][0][j] : qf[k][1][j - 4];
            const _Float16 h = (_Float16)x;
            h8[j] = h;
            l8[j] = (_Float16)(x - (float)h);
        }
        const int l = e & 63, c = (e >> 6) & 7, nt = e >> 9;
        *reinterpret_cast<half8 *>(Qs + (((nt * 2 + 0) * 8 + c) * 64 + l) * 16) = h8;
        *reinterpret_cast<half8 *>(Qs + (((nt * 2 + 1) * 8 + c) * 64 + l) * 16) = l8;
    }
    __syncthreads();
    // Bias table: the K bytes enter the MFMA as (b + 128) * 2^-24, so every score of block c
    // carries +128 * 2^-24 * sum_k q[k][n]; its negative is the C operand the block's MFMA starts
    // from.  One entry per (tile, block, column), replicated x4 for the accumulator layout.
    for (int e = threadIdx.x; e < NT * 8 * 16; e += kThreads) {
        const int n = e & 15, c = (e >> 4) & 7, nt = e >> 7;
        float sum = 0.0f;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const half8 h = *reinterpret_cast<const half8 *>(Qs + (((nt * 2 + 0) * 8 + c) * 64 + g * 16 + n) * 16);
            const half8 l = *reinterpret_cast<const half8 *>(Qs + (((nt * 2 + 1) * 8 + c) * 64 + g * 16 + n) * 16);
#pragma unroll
            for (int j = 0; j < 8; j++)
                sum += (float)h[j] + (float)l[j];
        }
        const float cb = -kOffset / kTwo24 * sum;
        *reinterpret_cast<float4v *>(CBs + ((nt * 8 + c) * 16 + n) * 16) = (float4v){cb, cb, cb, cb};
    }
    __syncthreads();

    // per-column causal bound (MTP rows see one more key each)
    int seq_n[NT];
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
        const int n = nt * 16 + lm;
        seq_n[nt] = n < nvalid ? seqc[n / group] : 0;
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

    // V transpose-read address: lane (2r+e) of its 16-lane group supplies key slot r
    // (slot r<4: key lg*4+r, slot r>=4: key 16+lg*4+(r-4)), bytes [8e, 8e+8) of a 16-d run.
    const int tr_r = lm >> 1;
    const int tr_key = (tr_r >> 2) * 16 + lg * 4 + (tr_r & 3);
    const uint8_t *vtr = tile_lds + tr_key * kLdsRow + (lm & 1) * 8;
    constexpr uint32_t kBiasBits = Q4 ? 0x80088008u : 0x80808080u;
    const uint4v bias_bits = {kBiasBits, kBiasBits, kBiasBits, kBiasBits};
    const half8 Abias = __builtin_bit_cast(half8, bias_bits); // eight times -offset * 2^-24

    auto process = [&](Unit (&Ku)[2], Unit (&Vu)[2], int t) {
        const int key0 = tile_key0(t);
        const bool more = t + 1 < ntile;

        // ---- K tile to LDS, refill the registers ------------------------------------------
        store_unit(Ku[0], tile_lds, sK, ur0, upr, key0 + ur0 < hi);
        store_unit(Ku[1], tile_lds, sK, ur1, upr, key0 + ur1 < hi);
        // (the refill sits under a branch, so the compiler cannot count the loads in flight and the
        // next use of an older load waits for all of them; issuing it unconditionally, with idle
        // addresses for a wave that has no further tile, gives exact waits and measured no faster:
        // 24.9 against 25.1 us at depth 32,768, 59.0 against 58.1 at 131,072, 80.5 against 78.7 on
        // the 16-slot batch)
        if (more)
            issue(Ku, kbase, t + 1);

        // ---- scores ------------------------------------------------------------------------
        float S[NT][2][4];
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
#pragma unroll
            for (int ms = 0; ms < 2; ms++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    S[nt][ms][i] = 0.0f;
#pragma unroll
        for (int c = 0; c < 8; c++) {
            half8 bh[NT], bl[NT];
            float4v cbias[NT];
#pragma unroll
            for (int nt = 0; nt < NT; nt++) {
                cbias[nt] = *reinterpret_cast<const float4v *>(CBs + ((nt * 8 + c) * 16 + lm) * 16);
                bh[nt] = *reinterpret_cast<const half8 *>(Qs + (((nt * 2 + 0) * 8 + c) * 64 + lane) * 16);
                bl[nt] = *reinterpret_cast<const half8 *>(Qs + (((nt * 2 + 1) * 8 + c) * 64 + lane) * 16);
            }
#pragma unroll
            for (int ms = 0; ms < 2; ms++) {
                const int2v raw = *reinterpret_cast<const int2v *>(
                    tile_lds + (ms * 16 + lm) * kLdsRow + c * 32 + lg * 8);
                const half8 A = bytes_to_f16_biased<Q4>(raw);
                const half4 sk = *reinterpret_cast<const half4 *>(
                    sK + (c * kTileKeys + ms * 16 + lg * 4) * 2);
#pragma unroll
                for (int nt = 0; nt < NT; nt++) {
                    float4v part = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, bh[nt], cbias[nt], 0, 0, 0);
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, bl[nt], part, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        S[nt][ms][i] = fmaf((float)sk[i], part[i], S[nt][ms][i]);
                }
            }
            // finish this block's scores here: left alone, the optimiser sinks all 8 blocks'
            // multiply-adds below the refill branch and keeps 16 MFMA results alive
#pragma unroll
            for (int nt = 0; nt < NT; nt++)
#pragma unroll
                for (int ms = 0; ms < 2; ms++)
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        PIN(S[nt][ms][i]);
        }

        // ---- V tile over the K tile, refill -----------------------------------------------
        store_unit(Vu[0], tile_lds, sV, ur0, upr, key0 + ur0 < hi);
        store_unit(Vu[1], tile_lds, sV, ur1, upr, key0 + ur1 < hi);
        if (more)
            issue(Vu, vbase, t + 1);

        // ---- online softmax (log2 units), per column n = lane%16 -----------------------
        // The probabilities are rounded to f16 once, here; the running sum uses the rounded
        // values, so numerator and denominator see the same weights.
        float p[NT][2][4];
        half4 ph[NT][2];
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
            mt = quad_rows<true>(mt);
            const float m_new = fmaxf(m_run[nt], mt);
            corr[nt] = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_run[nt] - m_new);
            grew = grew || (m_new > m_run[nt]);
            float ls = 0.0f;
#pragma unroll
            for (int ms = 0; ms < 2; ms++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float e = m_new == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(S[nt][ms][i] - m_new);
                    if (PLO) {
                        p[nt][ms][i] = e;
                        ls += e;
                    } else {
                        const _Float16 eh = (_Float16)e;
                        ph[nt][ms][i] = eh;
                        ls += (float)eh;
                    }
                }
            l_run[nt] = l_run[nt] * corr[nt] + ls;
            m_run[nt] = m_new;
        }
        if (__any(grew)) {
#pragma unroll
            for (int nt = 0; nt < NT; nt++)
#pragma unroll
                for (int t2 = 0; t2 < 16; t2++)
                    O[nt][t2] *= corr[nt];
        }

        // ---- O^T += V^T . P' ---------------------------------------------------------------
#pragma unroll
        for (int c = 0; c < 8; c++) {
            // rows past `hi` are duplicates of the last live row: finite scale, p = 0
            half4 sv[2];
#pragma unroll
            for (int ms = 0; ms < 2; ms++)
                sv[ms] = *reinterpret_cast<const half4 *>(sV + (c * kTileKeys + ms * 16 + lg * 4) * 2);
            // P' = p * block scale.  Default: one packed f16 multiply (f16-class weights);
            // PLO carries hi + lo f16 so the product keeps ~22 bits.
            half8 Ph[NT], Pl[NT];
#pragma unroll
            for (int nt = 0; nt < NT; nt++) {
                if (PLO) {
#pragma unroll
                    for (int ms = 0; ms < 2; ms++)
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const float x = p[nt][ms][i] * (float)sv[ms][i];
                            const _Float16 h = (_Float16)x;
                            Ph[nt][ms * 4 + i] = h;
                            Pl[nt][ms * 4 + i] = (_Float16)(x - (float)h);
                        }
                } else {
                    const half4 x0 = ph[nt][0] * sv[0];
                    const half4 x1 = ph[nt][1] * sv[1];
                    Ph[nt] = __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7);
                }
            }
#pragma unroll
            for (int hf = 0; hf < 2; hf++) {
                const int2v raw = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                    (int2v __attribute__((address_space(3))) *)(vtr + c * 32 + hf * 16));
                const half8 A = bytes_to_f16_biased<Q4>(raw);
#pragma unroll
                for (int nt = 0; nt < NT; nt++) {
                    float4v o = O[nt][c * 2 + hf];
                    o = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, Ph[nt], o, 0, 0, 0);
                    o = __builtin_amdgcn_mfma_f32_16x16x32_f16(Abias, Ph[nt], o, 0, 0, 0);
                    if (PLO) {
                        o = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, Pl[nt], o, 0, 0, 0);
                        o = __builtin_amdgcn_mfma_f32_16x16x32_f16(Abias, Pl[nt], o, 0, 0, 0);
                    }
                    O[nt][c * 2 + hf] = o;
                }
            }
        }
    };

    for (int t = 0; t < ntile; t++)
        process(Kst, Vst, t);

    // ---- merge the four waves and write the split's partial -------------------------------
    // O^T C layout: lane holds d = t*16 + lg*4 + i for column n = lane%16.  Rounds of 8 columns:
    // each wave parks 8 columns x 256 d (8 KiB) in its own tile area.
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
        l_run[nt] = quad_rows<false>(l_run[nt]);
    }
    float *wl = reinterpret_cast<float *>(tile_lds); // per wave: [8][256] acc
    float *wml = reinterpret_cast<float *>(sK);      // per wave: [8] m, [8] l
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const int nbase = nt * 16 + half * 8;
            if (nbase >= nvalid)
                break; // uniform over the workgroup
            __syncthreads(); // everyone is done with the tile buffers / previous round
            if ((lm >> 3) == half) {
                const int n8 = lm & 7;
#pragma unroll
                for (int t = 0; t < 16; t++)
                    *reinterpret_cast<float4v *>(wl + n8 * kHeadDim + t * 16 + lg * 4) = O[nt][t];
                if (lg == 0) {
                    wml[n8] = m_run[nt];
                    wml[8 + n8] = l_run[nt];
                }
            }
            __syncthreads();
            // thread -> (column n8, kRun consecutive d): 8 columns x kThreads/8 d-runs
            constexpr int kRuns = kThreads / 8, kRun = kHeadDim / kRuns;
            const int n8 = threadIdx.x / kRuns;
            const int d0 = (threadIdx.x % kRuns) * kRun;
            const int ng = nbase + n8;
            if (ng < nvalid) {
                float mw[kWaves], lw[kWaves];
                float ms = -INFINITY;
#pragma unroll
                for (int w = 0; w < kWaves; w++) {
                    const float *o = reinterpret_cast<const float *>(wave_base + w * kWaveLds + kTileBytes);
                    mw[w] = o[n8];
                    lw[w] = o[8 + n8];
                    ms = fmaxf(ms, mw[w]);
                }
                float lsum = 0.0f;
                float wgt[kWaves];
#pragma unroll
                for (int w = 0; w < kWaves; w++) {
                    wgt[w] = mw[w] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(mw[w] - ms);
                    lsum += lw[w] * wgt[w];
                    wgt[w] *= kTwo24;
                }
                const int col = ng / group;
                const int head = hbase + (ng - col * group);
                const size_t slice = (size_t)head * f.splits + split;
                float *pa = a.part_acc + (size_t)(row0 + col) * a.acc_slot + slice * kHeadDim + d0;
#pragma unroll
                for (int dd = 0; dd < kRun; dd += 4) {
                    float4v acc = {0, 0, 0, 0};
#pragma unroll
                    for (int w = 0; w < kWaves; w++) {
                        const float *o = reinterpret_cast<const float *>(wave_base + w * kWaveLds);
                        const float4v x = *reinterpret_cast<const float4v *>(o + n8 * kHeadDim + d0 + dd);
                        acc += x * wgt[w];
                    }
                    *reinterpret_cast<float4v *>(pa + dd) = acc;
                }
                if (threadIdx.x % kRuns == 0) {
                    float *pm = a.part_ml + (size_t)(row0 + col) * a.ml_slot + slice * 2;
                    pm[0] = ms;
                    pm[1] = lsum;
                }
            }
        }
    }
}

// The register-staged kernel: one 16-column tile per workgroup (wider slots arrive as several work
// items).  It serves q4_0 caches and, with PLO, the fp32-class variant of the q8_0 decode.
template <bool Q4, bool PLO>
__global__ void __launch_bounds__(kThreads, 2) decode_staged_kernel(const DecodeArgs a)
{
    decode_body<1, Q4, PLO>(a);
}

// ---------------------------------------------------------------------------------------------
// The q8_0 decode kernel.  Same work split, arithmetic and partial format as the staged kernel
// above, but the cache rows travel from memory straight into LDS (global_load_lds_dwordx4) and are
// used as they lie there, 272 bytes per key: no staging registers, no realignment, no LDS writes
// by the wave, and a refill is one scalar-addressed instruction per KiB.
//
//   K operand   lane (key lm, k-group lg) needs the 8 payload bytes of block c at
//               key*272 + 34c + 2 + 8 lg: two or three aligned dwords (raw_k_operand; the 272-byte
//               pitch spreads the 16 keys of a read over all banks).
//   V operand   ds_read_tr8_b64 wants 8-byte aligned addresses, and a block's payload starts
//               2 (mod 4) bytes into the row.  The rows of O^T may come in any order, though, so
//               the row is cut into its 17 aligned runs of 16 byte columns instead of 16 runs of
//               16 values of d: run j is one A operand, its 16 columns are scale bytes (rows that
//               are never read back) or values of d.  Six runs hold columns of two blocks, whose
//               weights p * block scale differ: they are multiplied once with each block's
//               weights, into two accumulators, and each column is taken from the one that
//               belongs to it at the end.  23 accumulators instead of 16, no data movement.
//   +128        the bytes enter as (b + 128) * 2^-24.  Scores: the MFMA of block c starts from
//               -128 * 2^-24 * sum of the block's Q values (a 2 KiB table in LDS).  PV: what has to
//               come off every row of block c is 128 * 2^-24 * sum_key P'_c[key][n], i.e. the row a
//               constant A operand of 128 * 2^-24 would produce.  The two scale-byte columns of block
//               c are such spare rows, and they sit in the first run of the block: their bytes are
//               replaced by the constant on the way to the MFMA, the row accumulates the correction
//               next to the data, and the merge subtracts column 34c from the block's columns.
//               (Block 7 has no scale byte in its own runs: one extra MFMA per tile.)
//   scales      a wave copies the 256 block scales of a tile into the transposed f16 table
//               [8 blocks][32 keys] (4 ds_read_u16 + 1 ds_write_b64 per lane) before it uses them.
//   Q           f16 B operands in registers (8 blocks x 4 registers); each wave fetches and converts
//               two of the blocks and the four exchange them through LDS.
//
// Pipeline of a wave: K rows of tile t+1 are requested as soon as the scores of tile t are done, V
// rows of tile t+1 after its PV product, so 8.7 to 17.4 KB per wave are in flight at any time.
// The loads are written as asm: the compiler then neither knows nor waits for them, and the waits
// are the explicit s_waitcnt below (loads return in order, 9 instructions per tile of rows).
constexpr int kRawTile = kTileKeys * kRowBytes;              // 8704: 32 key rows as they lie in the cache
constexpr int kParkPitch = kRowBytes + 4;                    // floats between parked accumulator rows (see the merge of the waves)
constexpr int kDmaTileLds = 16 * kParkPitch * 4;             // K rows and V rows of one tile (17,408 bytes), and room for a
                                                             // wave to park 16 columns of accumulators at the end (17,664)
static_assert(kDmaTileLds >= 2 * kRawTile, "a wave's K and V rows");
constexpr int kDmaQLds = 8 * 64 * 16;                        // Q operands on their way to registers: [8 blocks][64 lanes] half8;
                                                             // afterwards the waves' scale tables (2 x 512 bytes each)
constexpr int kDmaBiasLds = 8 * 16 * 16;                     // score bias: [8 blocks][16 columns] float4
// One tile of K and V rows per wave: 80,896 bytes, two workgroups per CU.  (A second tile per wave in
// LDS, for launches of one workgroup per CU, measured slower: 21.3 against 19.2 us at depth 32,768,
// as did a streaming probe with 16 instead of 8 KB in flight per wave.)
constexpr int kDmaLds = kWaves * kDmaTileLds + kDmaQLds + kDmaBiasLds;
constexpr int kRuns = kRowBytes / 16;                        // 17 runs of 16 byte columns
constexpr int kAccs = 23;                                    // 3 per block 0..6, 2 for block 7


__device__ __forceinline__ uint32_t lds_address(const void *p)
{
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}

// 64 lanes x 16 bytes from base + voff (per lane) to LDS address lds_at + 16 * lane.  ONCE: the
// rows are read by this launch once, so the load is non-temporal (streaming 71 MB that way measured
// 12.1 against 13.7 us per launch); rows that other work items of the launch read again are left
// to the L2's ordinary policy.
template <bool ONCE>
__device__ __forceinline__ void dma16(uint32_t lds_at, const uint8_t *base, uint32_t voff)
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

// Device-scope accesses to the split partials.  A workgroup that merges partials (decode_merge_tail) reads
// what workgroups on other XCDs, behind other L2 caches, have written while the same kernel runs.  A fence
// would make that safe by writing back and invalidating a whole L2, once per wave: measured, it turned a
// 19-us launch into one of 65 us.  Instead every access to a partial carries device scope itself (relaxed
// atomic accesses of 64 bits: stores that are acknowledged once they are visible to the whole device, loads
// that do not take a line another XCD may have changed from the local caches), and the order is kept by
// waiting for the stores' acknowledgements before the ticket is drawn.
__device__ __forceinline__ void store_dev(float *p, float2 v)
{
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(p), __builtin_bit_cast(unsigned long long, v),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_dev(float *p, float4v v)
{
    store_dev(p, (float2){v[0], v[1]});
    store_dev(p + 2, (float2){v[2], v[3]});
}
__device__ __forceinline__ float2 load_dev2(const float *p)
{
    return __builtin_bit_cast(float2, __hip_atomic_load(reinterpret_cast<const unsigned long long *>(p),
                                                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ float4v load_dev4(const float *p)
{
    const float2 a = load_dev2(p), b = load_dev2(p + 2);
    return (float4v){a.x, a.y, b.x, b.y};
}

// A operand of a score MFMA from a raw key row: the 8 payload bytes [8 lg, 8 lg + 8) of block c as
// f16 (b + 128) * 2^-24; `row_lg` = row + 8 lg.  LDS reads that are not aligned to their size run at a
// fraction of the rate of aligned ones (measured: 35-64 against 2-3 cycles per ds_read_b64 over the
// CU), so the bytes are taken from aligned dwords: two for an odd block (its payload starts at a dword),
// three for an even one (payload 2 bytes into a dword; the byte selects of the conversion do the shift).
__device__ __forceinline__ half8 raw_k_operand(const uint8_t *row_lg, int c)
{
    uint4v r;
    if (c & 1) {
        const uint32_t *p = reinterpret_cast<const uint32_t *>(row_lg + c * kQ8BlockBytes + 2);
        const uint32_t x0 = p[0] ^ 0x80808080u, x1 = p[1] ^ 0x80808080u;
        r[0] = __builtin_amdgcn_perm(0u, x0, 0x0c010c00u);
        r[1] = __builtin_amdgcn_perm(0u, x0, 0x0c030c02u);
        r[2] = __builtin_amdgcn_perm(0u, x1, 0x0c010c00u);
        r[3] = __builtin_amdgcn_perm(0u, x1, 0x0c030c02u);
    } else {
        const uint32_t *p = reinterpret_cast<const uint32_t *>(row_lg + c * kQ8BlockBytes);
        const uint32_t x0 = p[0] ^ 0x80808080u, x1 = p[1] ^ 0x80808080u, x2 = p[2] ^ 0x80808080u;
        r[0] = __builtin_amdgcn_perm(0u, x0, 0x0c030c02u);
        r[1] = __builtin_amdgcn_perm(0u, x1, 0x0c010c00u);
        r[2] = __builtin_amdgcn_perm(0u, x1, 0x0c030c02u);
        r[3] = __builtin_amdgcn_perm(0u, x2, 0x0c010c00u);
    }
    return __builtin_bit_cast(half8, r);
}

// The same for a q4_0 row: k-group lg of block c = the low (shift 0) or high (shift 4) nibbles of the 8 payload
// bytes [8 (lg & 1), + 8) of the block; `row_b` = row + 8 (lg & 1).  A payload starts 2 bytes into its 18-byte
// block: dword aligned in odd blocks, 2 bytes into a dword in even ones, as in a q8_0 row.  The nibble enters as
// n * 2^-24 (values n - 8: the offset comes off through the score bias, as the q8_0 offset of 128 does).
__device__ __forceinline__ half8 raw_k_operand_q4(const uint8_t *row_b, int c, int shift)
{
    uint4v r;
    if (c & 1) {
        const uint32_t *p = reinterpret_cast<const uint32_t *>(row_b + c * kQ4BlockBytes + 2);
        const uint32_t x0 = (p[0] >> shift) & 0x0f0f0f0fu, x1 = (p[1] >> shift) & 0x0f0f0f0fu;
        r[0] = __builtin_amdgcn_perm(0u, x0, 0x0c010c00u);
        r[1] = __builtin_amdgcn_perm(0u, x0, 0x0c030c02u);
        r[2] = __builtin_amdgcn_perm(0u, x1, 0x0c010c00u);
        r[3] = __builtin_amdgcn_perm(0u, x1, 0x0c030c02u);
    } else {
        const uint32_t *p = reinterpret_cast<const uint32_t *>(row_b + c * kQ4BlockBytes);
        const uint32_t x0 = (p[0] >> shift) & 0x0f0f0f0fu, x1 = (p[1] >> shift) & 0x0f0f0f0fu,
                       x2 = (p[2] >> shift) & 0x0f0f0f0fu;
        r[0] = __builtin_amdgcn_perm(0u, x0, 0x0c030c02u);
        r[1] = __builtin_amdgcn_perm(0u, x1, 0x0c010c00u);
        r[2] = __builtin_amdgcn_perm(0u, x1, 0x0c030c02u);
        r[3] = __builtin_amdgcn_perm(0u, x2, 0x0c010c00u);
    }
    return __builtin_bit_cast(half8, r);
}

// WIDE: the item has 9 to 16 (row, head) columns (rows of an MTP-verify slot).  Then every MFMA column
// is a real one, the two f16 halves of Q are two B operands and two MFMAs per block, and the raw Q rows
// (16 KB) pass through the waves' V rows before the first V rows are requested.
template <bool WIDE, bool Q4 = false>
__device__ __forceinline__ void decode_body_dma(const DecodeArgs &a, const Front &f, const Work &wk HIPML_STAMPS_ARG)
{
    static_assert(kWaves * 2 * kScaleBytes <= kDmaQLds, "the scale tables reuse the Q staging area");
    static_assert(!(WIDE && Q4), "q4_0 rows are served in items of at most 8 columns");
    constexpr int kCols = WIDE ? 16 : 8; // columns of an item
    // q4_0 (Q4): a row is 144 bytes = 9 aligned 16-byte runs, a tile of 32 rows 4,608 bytes = 4.5 requests of
    // 1 KiB; byte j of a block holds element j in its low and element j + 16 in its high nibble
    // (crates/hipml-core/src/kv.rs:201-218), values n - 8.
    constexpr int kRowB = Q4 ? kRowBytesQ4 : kRowBytes;
    constexpr int kBlkB = Q4 ? kQ4BlockBytes : kQ8BlockBytes;
    constexpr int kRawT = kTileKeys * kRowB;     // 8,704 / 4,608: one tile of rows as they lie in the cache
    constexpr int kReq = Q4 ? 5 : 9;             // requests per tile of rows (the last one half a wave)
    constexpr int kDmaWaveLds = kDmaTileLds;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_all[];
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int lm = lane & 15; // MFMA row/col within the 16-tile
    const int lg = lane >> 4; // k-group
    const int kvh = wk.kvh, split = wk.split, nsp = wk.nsp, slot = wk.slot, row0 = wk.row0, ncols = wk.ncols,
              group = wk.group, hbase = wk.hbase, nvalid = wk.nvalid;

    uint8_t *wave_lds = lds_all + wave * kDmaWaveLds;
    uint8_t *Kraw = wave_lds;
    uint8_t *Vraw = wave_lds + kRawT;
    uint8_t *Qst = lds_all + kWaves * kDmaWaveLds;
    uint8_t *CBs = Qst + kDmaQLds;
    uint8_t *sK = Qst + wave * 2 * kScaleBytes;
    uint8_t *sV = sK + kScaleBytes;
    const uint32_t wave_at = lds_address(wave_lds);

    // (a launch with one item gets its cache pointers at that item's slot: nothing to fetch for the address)
    const size_t slot_at = f.items == 1 ? 0 : (size_t)slot * a.kv_slot_bytes;
    const uint8_t *kbase = f.k + slot_at + (size_t)kvh * f.stride * kRowB;
    const uint8_t *vbase = f.v + slot_at + (size_t)kvh * f.stride * kRowB;

    // tile g of a KV head belongs to split (g / kWaves) % nsp, wave g % kWaves (see the staged kernel)
    auto tile_key0 = [&](int t) { return ((t * nsp + split) * kWaves + wave) * kTileKeys; };

    // ---- one tile of rows = 8,704 contiguous bytes = 8.5 instructions of 1 KiB ------------------
    const uint32_t lane16 = lane * 16;
    const uint32_t region_last = (uint32_t)f.stride * kRowB - 16; // last 16 bytes of a KV head's rows
    auto issue_as = [&](auto once, auto first, bool v_rows, int t) {
        constexpr bool kOnce = decltype(once)::value;
        const uint32_t lds_at = wave_at + (v_rows ? kRawT : 0);
        const uint8_t *region = v_rows ? vbase : kbase;
        const int key0 = tile_key0(t);
        // the wave's own reads of the old rows are done (the launch's first request replaces nothing, and a
        // wait here would be one for the live lengths, whose scalar loads count on the same counter)
        if (!decltype(first)::value)
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (key0 + kTileKeys <= f.stride) { // (uniform) the tile lies inside the cache
            const uint8_t *src = region + (size_t)key0 * kRowB;
#pragma unroll
            for (int j = 0; j < kReq - 1; j++)
                dma16<kOnce>(lds_at + j * 1024, src + j * 1024, lane16);
            if (lane < 32)
                dma16<kOnce>(lds_at + (kReq - 1) * 1024, src + (kReq - 1) * 1024, lane16);
        } else {
            // the last rows of the cache: bytes past its end are replaced by its last 16 (rows at or
            // past the live length are masked whatever they hold)
            const uint32_t off0 = (uint32_t)key0 * kRowB + lane16;
#pragma unroll
            for (int j = 0; j < kReq - 1; j++) {
                const uint32_t o = off0 + j * 1024;
                dma16<kOnce>(lds_at + j * 1024, region, o < region_last ? o : region_last);
            }
            if (lane < 32) {
                const uint32_t o = off0 + (kReq - 1) * 1024;
                dma16<kOnce>(lds_at + (kReq - 1) * 1024, region, o < region_last ? o : region_last);
            }
        }
    };
    // (an item that carries every head of its KV head is its slot's only reader of these rows)
    const bool once = f.stream_once != 0 || group == f.group;
    auto issue = [&](bool v_rows, int t) {
        if (once)
            issue_as(std::true_type(), std::false_type(), v_rows, t);
        else
            issue_as(std::false_type(), std::false_type(), v_rows, t);
    };
    auto issue_first = [&] {
        if (once)
            issue_as(std::true_type(), std::true_type(), false, 0);
        else
            issue_as(std::false_type(), std::true_type(), false, 0);
    };

    // live lengths of this slot's rows: lane c asks for that of row row0 + c with the launch's first vector load,
    // written out so that the wait is this code's own.  Requests return in order, so the wait for the Q rows
    // below is the wait for this one as well.  (As scalar loads they took 2 us to come back under the launch's
    // first burst, and every wait for an LDS read is one for outstanding scalar loads too: the Q conversion
    // stood behind them.  Left to the compiler, a vector load would be waited for with vmcnt(0): it does not
    // count the requests made in asm statements.)
    int pos_lane;
    {
        const int32_t *pp = f.pos + (size_t)(row0 + (lane < ncols ? lane : 0)) * 2 + 1;
        asm volatile("global_load_dword %0, %1, off" : "=v"(pos_lane) : "v"(pp) : "memory");
    }

    // ---- the first requests: the Q rows, then the K rows of tile 0 ------------------------------
    // No address here needs anything from device memory (a tile past the live rows costs one load of
    // rows inside the cache and is masked out), so these 11 requests leave before the first wait.
    // The item has at most 8 (row, head) columns.  MFMA column lm < 8 carries the f16 value of Q column
    // lm, MFMA column lm + 8 what that rounding left over (x - f16(x), again as f16): the two halves
    // of a score are added after the block loop, so Q enters with ~22 bits at the price of one
    // MFMA.  Wave w fetches two blocks of the Q rows, 2 KB, and the four exchange the operands made
    // of them through LDS below.  (Every wave fetching all of it is 16 KB per wave through the CU's L1
    // in front of the first K/V rows: 1 us later first data.)  The Q rows take the same road as the
    // K/V rows, global memory -> LDS, into the quarter of the staging area that the wave's operands
    // go to afterwards: written as ordinary loads they would be waited for by the compiler with
    // vmcnt(0), that is together with the K and V rows of tile 0 behind them.
    // Request i of lane l brings 16 bytes: column l % 8, block 2w + i, k-group (l / 8) % 4, half l / 32.
    constexpr int kQB = 8 / kWaves; // Q blocks per wave
    static_assert(kQB == 2, "two requests of 64 x 16 bytes fetch a wave's share of the Q rows of 8 columns");
    const int qcol = WIDE ? lm : lm & 7;
    const bool have_q = qcol < nvalid;
    // WIDE: four requests per wave (16 columns) into the wave's V rows, whose first tile is requested
    // once the values are in registers; request i of lane l: column l % 16, block 2w + i / 2,
    // k-group l / 16, half i % 2, so every lane finds its own values in its own slots.
    uint8_t *Qraw = WIDE ? Vraw : Qst + wave * (kQB * 1024);
    {
        const int lcol = WIDE ? (lane & 15) : (lane & 7);
        const int fcol = lcol < nvalid ? lcol : 0; // (idle columns fetch column 0 and drop it)
        const int col = fcol / group;
        const int head = fcol - col * group;
        const int kg = WIDE ? (lane >> 4) : ((lane >> 3) & 3);
        // (per-lane byte offsets from the uniform base: the Q rows of a launch are far below 4 GB)
        const uint32_t qoff = (uint32_t)(((size_t)(row0 + col) * f.q_slot + (size_t)(hbase + head) * kHeadDim +
                                          wave * (kQB * 32) + kg * 8 + (WIDE ? 0 : (lane >> 5) * 4)) *
                                         sizeof(float));
        const uint32_t at = lds_address(Qraw);
        const uint8_t *qb = reinterpret_cast<const uint8_t *>(f.q);
        if (WIDE) {
#pragma unroll
            for (int i = 0; i < 4; i++)
                dma16<false>(at + i * 1024, qb, qoff + ((i >> 1) * 32 + (i & 1) * 4) * sizeof(float));
        } else {
            dma16<false>(at, qb, qoff);
            dma16<false>(at + 1024, qb, qoff + 32 * sizeof(float));
        }
    }
    issue_first();
    HIPML_STAMP(stamps_, 2); // the first requests have left

    // all but the newest tile of rows have arrived (requests return in the order of issue)
    auto wait_all_but_one_tile = [] {
        if (Q4)
            asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
        else
            asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
    };
    // the Q rows are in LDS, and the live lengths in their register, once only the requests behind them are
    // outstanding: K(0)
    if (Q4)
        asm volatile("s_waitcnt vmcnt(5)" : "+v"(pos_lane) : : "memory");
    else
        asm volatile("s_waitcnt vmcnt(9)" : "+v"(pos_lane) : : "memory");
    int seqc[kMaxCols];
    int seq_max = 0;
#pragma unroll
    for (int c = 0; c < kMaxCols; c++) {
        int s = c < ncols ? __builtin_amdgcn_readlane(pos_lane, c) : 0;
        s = s < 0 ? 0 : (s > f.stride ? f.stride : s);
        seqc[c] = s;
        seq_max = s > seq_max ? s : seq_max;
    }
    const int hi = seq_max; // keys at or past it are masked
    if (split * kWaves * kTileKeys >= hi) {
        // not one live tile for any wave of this workgroup: leave an empty partial, which the merge skips
        if ((int)threadIdx.x < nvalid) {
            const int col = threadIdx.x / group;
            const int head = hbase + (threadIdx.x - col * group);
            float *pm = a.part_ml + (size_t)(row0 + col) * a.ml_slot + ((size_t)head * f.splits + split) * 2;
            store_dev(pm, (float2){-INFINITY, 0.0f});
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // nothing may land in LDS after the wave has gone
        return; // uniform over the workgroup
    }
    const int first_key = tile_key0(0), step_keys = nsp * kWaves * kTileKeys;
    const int ntile = first_key < hi ? (hi - first_key + step_keys - 1) / step_keys : 0;

    // ---- Q operands and the score bias of every block ------------------------------------------
    float4v qf[kQB][2];
#pragma unroll
    for (int cc = 0; cc < kQB; cc++)
#pragma unroll
        for (int h = 0; h < 2; h++)
            qf[cc][h] = WIDE ? *reinterpret_cast<const float4v *>(Qraw + (cc * 2 + h) * 1024 + lane * 16)
                             : *reinterpret_cast<const float4v *>(Qraw + cc * 1024 + ((h << 5) | (lg << 3) | qcol) * 16);
    half8 qlo[kQB]; // WIDE: what the rounding to f16 left over, the second B operand
#pragma unroll
    for (int cc = 0; cc < kQB; cc++) {
        const int c = kQB * wave + cc;
        half8 h8;
        float sum = 0.0f, sum_lo = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float x = have_q ? (j < 4 ? qf[cc][0][j] : qf[cc][1][j - 4]) : 0.0f;
            _Float16 h = (_Float16)x;
            const _Float16 l = (_Float16)(x - (float)h);
            if (WIDE) {
                qlo[cc][j] = l;
                sum_lo += (float)l;
            } else if (lm >= 8) {
                h = l;
            }
            sum += (float)h;
            h8[j] = h;
        }
        sum = quad_rows<false>(sum); // over the four k-groups: the block's 32 values of MFMA column lm
        const float cb = (Q4 ? -8.0f : -128.0f) / kTwo24 * sum; // the offset the K bytes (nibbles) carry
        // (narrow: the wave's own quarter: every lane has read its raw values, LDS works in program order)
        *reinterpret_cast<half8 *>(Qst + (c * 64 + lane) * 16) = h8;
        if (WIDE) {
            // both halves' biases side by side: every sum is formed as the narrow variant forms it in
            // its two column halves, so a column's result does not depend on the width of its item
            sum_lo = quad_rows<false>(sum_lo);
            const float cbl = -128.0f / kTwo24 * sum_lo;
            if (lg == 0)
                *reinterpret_cast<float4v *>(CBs + (c * 16 + lm) * 16) = (float4v){cb, cbl, 0.0f, 0.0f};
        } else if (lg == 0) {
            *reinterpret_cast<float4v *>(CBs + (c * 16 + lm) * 16) = (float4v){cb, cb, cb, cb};
        }
    }
    // The V rows of tile 0 are requested only now.  Asked for together with the K rows they make the launch's
    // first burst 18 MB, which the memory pipeline takes 3 us to accept: the waves sat in those requests while
    // their Q rows had long arrived, and the first scores, and with them the request for the next K rows, came
    // that much later (measured: 18.4 against 19.0 us per layer at depth 32,768, 10.3 against 10.9 at 8,192).
    // (WIDE: the raw Q values have left the V rows by now.)
    issue(true, 0);
    __syncthreads();
    half8 bh[8], bl[WIDE ? 8 : 1];
#pragma unroll
    for (int c = 0; c < 8; c++)
        bh[c] = *reinterpret_cast<const half8 *>(Qst + (c * 64 + lane) * 16);
    __syncthreads();
    if (WIDE) {
#pragma unroll
        for (int cc = 0; cc < kQB; cc++)
            *reinterpret_cast<half8 *>(Qst + ((kQB * wave + cc) * 64 + lane) * 16) = qlo[cc];
        __syncthreads();
#pragma unroll
        for (int c = 0; c < 8; c++)
            bl[WIDE ? c : 0] = *reinterpret_cast<const half8 *>(Qst + (c * 64 + lane) * 16);
        __syncthreads();
    }
    // (the staging area is the waves' scale tables from here on)
    HIPML_STAMP(stamps_, 3); // Q operands in registers

    // per-column causal bound (MTP rows see one more key each)
    const int seq_n = qcol < nvalid ? seqc[qcol / group] : 0;

    // ---- running state ----------------------------------------------------------------------
    float m_run = -INFINITY, l_run = 0.0f;
    // q8_0: 23 accumulators over the 17 runs of a row (see above); q4_0: two per run of its 9, low and high nibbles
    constexpr int kNAcc = Q4 ? 18 : kAccs;
    float4v O[kNAcc], B7 = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < kNAcc; i++)
        O[i] = (float4v){0, 0, 0, 0};

    // V transpose-read address: lane (2r+e) of its 16-lane group supplies key slot r
    // (slot r<4: key lg*4+r, slot r>=4: key 16+lg*4+(r-4)), bytes [8e, 8e+8) of a 16-column run.
    const int tr_r = lm >> 1;
    const int tr_key = (tr_r >> 2) * 16 + lg * 4 + (tr_r & 3);
    const uint8_t *vtr = Vraw + tr_key * kRowB + (lm & 1) * 8;
    // q4_0: the block that byte column 16 j + lm of run j belongs to (its scales go with this lane's rows of V^T),
    // as the offset of that block's 32 scales in the table
    int q4_scale_at[Q4 ? 9 : 1];
    if (Q4) {
#pragma unroll
        for (int j = 0; j < 9; j++)
            q4_scale_at[Q4 ? j : 0] = ((16 * j + lm) * 3641 >> 16) * (kTileKeys * 2); // (x / 18 for x < 144)
    }
    const uint4v bias_bits = {0x00800080u, 0x00800080u, 0x00800080u, 0x00800080u};
    const half8 Abias = __builtin_bit_cast(half8, bias_bits); // eight times 128 * 2^-24
    const int lm2 = lm >> 1; // run 2c carries the scale bytes of block c in rows 2c and 2c+1

    // the scales of a tile of raw rows -> f16 table [8 blocks][32 keys]; lane = (block, four keys)
    const int sc_c = lane >> 3, sc_k = (lane & 7) * 4;
    auto build_scales = [&](const uint8_t *raw, uint8_t *table, int key0, bool partial) {
        const uint8_t *p = raw + sc_k * kRowB + sc_c * kBlkB;
        uint32_t s0 = *reinterpret_cast<const uint16_t *>(p);
        uint32_t s1 = *reinterpret_cast<const uint16_t *>(p + kRowB);
        uint32_t s2 = *reinterpret_cast<const uint16_t *>(p + 2 * kRowB);
        uint32_t s3 = *reinterpret_cast<const uint16_t *>(p + 3 * kRowB);
        if (partial) {
            // a row at or past the live length holds whatever the cache holds there: zero scale, so
            // that its zero weight cannot meet a non-finite value
            const int k = key0 + sc_k;
            s0 = k < hi ? s0 : 0u;
            s1 = k + 1 < hi ? s1 : 0u;
            s2 = k + 2 < hi ? s2 : 0u;
            s3 = k + 3 < hi ? s3 : 0u;
        }
        int2v w;
        w[0] = (int)(s0 | (s1 << 16));
        w[1] = (int)(s2 | (s3 << 16));
        *reinterpret_cast<int2v *>(table + (sc_c * kTileKeys + sc_k) * 2) = w;
    };

    for (int t = 0; t < ntile; t++) {
        const int key0 = tile_key0(t);
        const bool more = t + 1 < ntile;
        const bool partial = key0 + kTileKeys > hi;
        // Requests complete in the order of issue, 9 per tile of rows: K(0) V(0), then K(t + 1) after the
        // scores of tile t and V(t + 1) after its PV.
        // ---- K rows of this tile are in LDS once only the loads of its V rows are outstanding
        wait_all_but_one_tile();
#ifdef HIPML_DECODE_STAMPS
        if (t == 0)
            HIPML_STAMP(stamps_, 4); // K rows of the wave's first tile in LDS
#endif
        build_scales(Kraw, sK, key0, partial);

        // ---- scores ----------------------------------------------------------------------------
        float S[2][4], Sl[WIDE ? 2 : 1][4]; // (Sl: the scores' lower halves where they have no columns of their own)
#pragma unroll
        for (int ms = 0; ms < 2; ms++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                S[ms][i] = Sl[WIDE ? ms : 0][i] = 0.0f;
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const float4v cb4 = *reinterpret_cast<const float4v *>(CBs + (c * 16 + lm) * 16);
#pragma unroll
            for (int ms = 0; ms < 2; ms++) {
                const half8 A = Q4 ? raw_k_operand_q4(Kraw + (ms * 16 + lm) * kRowB + (lg & 1) * 8, c, (lg >> 1) * 4)
                                   : raw_k_operand(Kraw + (ms * 16 + lm) * kRowB + lg * 8, c);
                const half4 sk = *reinterpret_cast<const half4 *>(sK + (c * kTileKeys + ms * 16 + lg * 4) * 2);
                if (WIDE) {
                    const float4v ch = {cb4[0], cb4[0], cb4[0], cb4[0]}, cl = {cb4[1], cb4[1], cb4[1], cb4[1]};
                    const float4v part = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, bh[c], ch, 0, 0, 0);
                    const float4v parl = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, bl[WIDE ? c : 0], cl, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        S[ms][i] = fmaf((float)sk[i], part[i], S[ms][i]);
                        Sl[WIDE ? ms : 0][i] = fmaf((float)sk[i], parl[i], Sl[WIDE ? ms : 0][i]);
                    }
                } else {
                    const float4v part = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, bh[c], cb4, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        S[ms][i] = fmaf((float)sk[i], part[i], S[ms][i]);
                }
            }
        }
        // the two halves of every score: MFMA columns n and n + 8 (a rotation by 8 inside the 16-lane
        // row), or the second set of sums
#pragma unroll
        for (int ms = 0; ms < 2; ms++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if (WIDE)
                    S[ms][i] += Sl[WIDE ? ms : 0][i];
                else
                    S[ms][i] += __builtin_bit_cast(
                        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, S[ms][i]), 0x128, 0xf, 0xf, true));
            }
        if (WIDE) {
            // (a fixed point for the instruction scheduler where the other variant has its lane moves:
            // without one it spreads the block loop over the softmax and runs out of registers)
            asm volatile("" : "+v"(S[0][0]), "+v"(S[0][1]), "+v"(S[0][2]), "+v"(S[0][3]), "+v"(S[1][0]), "+v"(S[1][1]),
                         "+v"(S[1][2]), "+v"(S[1][3]));
        }
        // the K rows are used up: request those of the tile that takes their place
        if (more)
            issue(false, t + 1);

        // ---- online softmax (log2 units), per column n = lane%16 -----------------------
        // The probabilities are rounded to f16 once, here; the running sum uses the rounded
        // values, so numerator and denominator see the same weights.
        half4 ph[2];
        float corr;
        bool grew;
        {
            const int lim = hi < seq_n ? hi : seq_n;
            float mt = -INFINITY;
#pragma unroll
            for (int ms = 0; ms < 2; ms++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int key = key0 + ms * 16 + lg * 4 + i;
                    const float s = key < lim ? S[ms][i] * a.scale_log2 : -INFINITY;
                    S[ms][i] = s;
                    mt = fmaxf(mt, s);
                }
            mt = quad_rows<true>(mt);
            // The reference value of the exponentials is not the running maximum: it moves only when
            // the maximum has passed it by more than 8 (log2 units), and then to 4 below the new
            // maximum.  Weights stay below 2^8, far inside f16 and f32; the 92 accumulator registers
            // are rescaled on a few tiles instead of most; and the small weights keep 4 to 8 more
            // bits above the f16 underflow than they would against the maximum itself.
            grew = mt > m_run + 8.0f;
            const float m_new = grew ? mt - 4.0f : m_run;
            corr = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
            float ls = 0.0f;
#pragma unroll
            for (int ms = 0; ms < 2; ms++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float e = m_new == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(S[ms][i] - m_new);
                    const _Float16 eh = (_Float16)e;
                    ph[ms][i] = eh;
                    ls += (float)eh;
                }
            l_run = l_run * corr + ls;
            m_run = m_new;
        }
        if (t > 0 && __any(grew)) { // (the accumulators of the first tile are still zero)
#pragma unroll
            for (int i = 0; i < kNAcc; i++)
                O[i] *= corr;
            B7 *= corr;
        }

        // ---- V rows of this tile: all that may still be outstanding are the next tile's K rows
        if (more)
            wait_all_but_one_tile();
        else
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#ifdef HIPML_DECODE_STAMPS
        if (!more)
            HIPML_STAMP(stamps_, 5); // V rows of the wave's last tile in LDS
#endif
        build_scales(Vraw, sV, key0, partial);

        // ---- O^T += V^T . P' -------------------------------------------------------------------
        if constexpr (Q4) {
            // One transposing read per run gives this lane the bytes of 8 keys in byte column 16 j + lm: their low
            // nibbles are a row of V^T (element e of the column's block), their high nibbles another (e + 16).
            // The block scale differs between the columns of a run, so it goes into the A operand: nibble n as
            // the f16 1024 + n, minus 1032 (exact), times the key's scale of the column's block (one rounding,
            // where the q8_0 path rounds the weight times the scale); P stays the plain f16 weights.  Columns
            // that hold scale bytes make rows nobody reads.
            const half8 Pp = __builtin_shufflevector(ph[0], ph[1], 0, 1, 2, 3, 4, 5, 6, 7);
            const half2v k1032 = {(_Float16)1032.0f, (_Float16)1032.0f};
#pragma unroll
            for (int j = 0; j < 9; j++) {
                const int2v raw = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                    (int2v __attribute__((address_space(3))) *)(vtr + j * 16));
                const half4 s0 = *reinterpret_cast<const half4 *>(sV + q4_scale_at[Q4 ? j : 0] + lg * 8);
                const half4 s1 = *reinterpret_cast<const half4 *>(sV + q4_scale_at[Q4 ? j : 0] + (16 + lg * 4) * 2);
                const half2v sc[4] = {{s0[0], s0[1]}, {s0[2], s0[3]}, {s1[0], s1[1]}, {s1[2], s1[3]}};
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const uint32_t y0 = ((uint32_t)raw[0] >> (4 * h)) & 0x0f0f0f0fu;
                    const uint32_t y1 = ((uint32_t)raw[1] >> (4 * h)) & 0x0f0f0f0fu;
                    uint4v r;
                    r[0] = __builtin_amdgcn_perm(0x64646464u, y0, 0x04010400u);
                    r[1] = __builtin_amdgcn_perm(0x64646464u, y0, 0x04030402u);
                    r[2] = __builtin_amdgcn_perm(0x64646464u, y1, 0x04010400u);
                    r[3] = __builtin_amdgcn_perm(0x64646464u, y1, 0x04030402u);
                    half8 A;
#pragma unroll
                    for (int w = 0; w < 4; w++) {
                        const uint32_t bits = r[w]; // (a copy: bit_cast of a vector element reads element 0)
                        const half2v x = (__builtin_bit_cast(half2v, bits) - k1032) * sc[w];
                        A[2 * w] = x[0];
                        A[2 * w + 1] = x[1];
                    }
                    O[2 * j + h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, Pp, O[2 * j + h], 0, 0, 0);
                }
            }
        } else {
            half8 Aprev = Abias; // the run shared with the previous block
    #pragma unroll
            for (int c = 0; c < 8; c++) {
                half4 sv[2];
    #pragma unroll
                for (int ms = 0; ms < 2; ms++)
                    sv[ms] = *reinterpret_cast<const half4 *>(sV + (c * kTileKeys + ms * 16 + lg * 4) * 2);
                // P' = p * block scale, one packed f16 multiply (f16-class weights)
                const half4 x0 = ph[0] * sv[0];
                const half4 x1 = ph[1] * sv[1];
                const half8 Ph = __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7);
                if (c == 7)
                    B7 = __builtin_amdgcn_mfma_f32_16x16x32_f16(Abias, Ph, B7, 0, 0, 0);
                // the runs that hold columns of block c: 2c .. 2c+2 (15 and 16 for block 7)
    #pragma unroll
                for (int r = 0; r < (c < 7 ? 3 : 2); r++) {
                    const int j = (c < 7 ? 2 * c : 15) + r;
                    half8 A;
                    if (r == 0 && c > 0 && c < 7) {
                        A = Aprev;
                    } else {
                        int2v raw = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                            (int2v __attribute__((address_space(3))) *)(vtr + j * 16));
                        if ((j & 1) == 0 && j <= 12) {
                            // rows j and j+1 of this run are scale bytes: byte 0 enters as 128 * 2^-24
                            raw[0] = lm2 == j / 2 ? 0 : raw[0];
                            raw[1] = lm2 == j / 2 ? 0 : raw[1];
                        }
                        A = bytes_to_f16_biased<false>(raw);
                    }
                    O[c * 3 + r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, Ph, O[c * 3 + r], 0, 0, 0);
                    if (r == 2)
                        Aprev = A;
                }
            }
        }
        // the V rows are used up
        if (more)
            issue(true, t + 1);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // (a wave without a tile still has its first K rows in flight)
    HIPML_STAMP(stamps_, 6); // the wave's last tile is done

    // ---- merge the four waves and write the split's partial -------------------------------
    // Run j of O^T: lane holds byte columns 16j + lg*4 + i of the key rows for column n = lane%16.
    // Each wave parks the item's columns as kCols x 272 values, indexed by byte column, in its own
    // rows (8 columns fill the K rows, 16 the K and V rows) and its (m, l) pairs in its own scale
    // table, so nothing has to be waited for before the writes; the other waves read them after the
    // barrier.
    l_run = quad_rows<false>(l_run);
    // The parked rows are 276 floats apart, so that the sixteen lanes of a k-group cover all 64 banks once
    // per 128-bit write (20 n mod 64 is a different multiple of 4 for each of 16 columns n).  With 8
    // columns the lanes of MFMA columns 8..15, which hold the same values as columns 0..7, write the run
    // ten further on, which lands in the other half of the banks (measured for four waves parking at
    // once: 470 cycles against 1,360 with rows of 272 floats written by half the lanes).
    float *wl = reinterpret_cast<float *>(wave_lds); // per wave: [kCols][kParkPitch] acc by byte column
    float *wml = reinterpret_cast<float *>(sK);  // per wave: [kCols] m, [kCols] l
    {
        auto run_values = [&](int j) {
            float4v v;
            if (j >= 2 && j <= 12 && (j & 1) == 0) {
                // columns of blocks j/2 - 1 (below byte 34 * (j/2)) and j/2
                const int c1 = j / 2;
                const float4v lo = O[3 * c1 - 1];
                const float4v up = O[3 * c1];
#pragma unroll
                for (int i = 0; i < 4; i++)
                    v[i] = 16 * j + lg * 4 + i < kQ8BlockBytes * c1 ? lo[i] : up[i];
            } else {
                const int idx = j == 0 ? 0 : (j >= 14 ? j + 6 : 3 * (j - 1) / 2 + 1);
                v = O[idx];
                if (j == 14) // byte column 238, the scale of block 7: its correction row
                    v[2] = lg == 3 ? B7[2] : v[2];
            }
            return v;
        };
        const int pc = lm & (kCols - 1); // the column this lane parks
        // q4_0: a column's rows are two halves of 144 byte columns (low nibbles, high nibbles), 160 floats apart,
        // columns 324 floats apart: the lanes of MFMA columns 0..7 write the low halves, those of columns 8..15
        // (the same values) the high halves, and the sixteen lanes of a k-group cover all 64 banks once per
        // 128-bit write (4 n mod 64 for n < 8, + 32 for the other half).
        constexpr int kQ4Half = 160, kQ4Pitch = 2 * kQ4Half + 4;
        static_assert(!Q4 || kCols * kQ4Pitch * 4 <= kDmaWaveLds, "a wave parks its columns in its own rows");
        if constexpr (Q4) {
            const bool first = lm < 8;
#pragma unroll
            for (int j = 0; j < 9; j++) {
                const float4v lo = O[Q4 ? 2 * j : 0], up = O[Q4 ? 2 * j + 1 : 0];
                const float4v v = {first ? lo[0] : up[0], first ? lo[1] : up[1], first ? lo[2] : up[2],
                                   first ? lo[3] : up[3]};
                *reinterpret_cast<float4v *>(wl + pc * kQ4Pitch + (first ? 0 : kQ4Half) + j * 16 + lg * 4) = v;
            }
        } else if (WIDE) {
#pragma unroll
            for (int j = 0; j < kRuns; j++)
                *reinterpret_cast<float4v *>(wl + pc * kParkPitch + j * 16 + lg * 4) = run_values(j);
        } else {
            static_assert(kRuns == 17, "runs j and j + 10 for j < 7, 7 and 9, and 8 alone");
            const bool first = lm < 8;
#pragma unroll
            for (int j = 0; j < 9; j++) {
                const int jp = j < 7 ? j + 10 : 9;
                const float4v a4 = run_values(j);
                if (j < 8) {
                    const float4v b4 = run_values(jp);
                    const float4v v = {first ? a4[0] : b4[0], first ? a4[1] : b4[1], first ? a4[2] : b4[2],
                                       first ? a4[3] : b4[3]};
                    *reinterpret_cast<float4v *>(wl + pc * kParkPitch + (first ? j : jp) * 16 + lg * 4) = v;
                } else if (first) {
                    *reinterpret_cast<float4v *>(wl + pc * kParkPitch + j * 16 + lg * 4) = a4;
                }
            }
        }
        if ((WIDE || lm < 8) && lg == 0) {
            wml[pc] = m_run;
            wml[kCols + pc] = l_run;
        }
        __syncthreads();
        // thread -> (column nc, kRun consecutive d of one block): kCols columns x kThreads / kCols runs of d
        constexpr int kDRuns = kThreads / kCols, kRun = kHeadDim / kDRuns;
        static_assert(kRun == 16 || kRun == 8, "a thread's values of d lie in one block");
        const int nc = threadIdx.x / kDRuns;
        const int d0 = (threadIdx.x % kDRuns) * kRun;
        // byte column of d0: 34 bytes per 32 values, scale first; q4_0: 18 bytes per 32 values, element e < 16 in
        // the low half at byte e, element e + 16 in the high half at the same byte
        const int col0 = Q4 ? (d0 >> 5) * kQ4BlockBytes + 2 + (d0 & 15) + ((d0 >> 4) & 1) * kQ4Half
                            : d0 + 2 + 2 * (d0 >> 5);
        if (nc < nvalid) {
            float mw[kWaves], lw[kWaves];
            float ms = -INFINITY;
#pragma unroll
            for (int w = 0; w < kWaves; w++) {
                const float *o = reinterpret_cast<const float *>(Qst + w * 2 * kScaleBytes);
                mw[w] = o[nc];
                lw[w] = o[kCols + nc];
                ms = fmaxf(ms, mw[w]);
            }
            float lsum = 0.0f;
            float wgt[kWaves];
#pragma unroll
            for (int w = 0; w < kWaves; w++) {
                wgt[w] = mw[w] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(mw[w] - ms);
                lsum += lw[w] * wgt[w];
                if (!Q4)
                    wgt[w] *= kTwo24; // (the q8_0 V operands carry 2^-24; the q4_0 ones are real values)
            }
            const int col = nc / group;
            const int head = hbase + (nc - col * group);
            const size_t slice = (size_t)head * f.splits + split;
            float *pa = a.part_acc + (size_t)(row0 + col) * a.acc_slot + slice * kHeadDim + d0;
#pragma unroll
            for (int dd = 0; dd < kRun; dd += 4) {
                float4v acc = {0, 0, 0, 0};
#pragma unroll
                for (int w = 0; w < kWaves; w++) {
                    const float *row = reinterpret_cast<const float *>(lds_all + w * kDmaWaveLds) +
                                       nc * (Q4 ? kQ4Pitch : kParkPitch);
                    const float off = Q4 ? 0.0f : row[(d0 >> 5) * kQ8BlockBytes]; // the block's correction row
                    const float2 x0 = *reinterpret_cast<const float2 *>(row + col0 + dd);
                    const float2 x1 = *reinterpret_cast<const float2 *>(row + col0 + dd + 2);
                    acc += ((float4v){x0.x, x0.y, x1.x, x1.y} - off) * wgt[w];
                }
                if (a.merge > 0)
                    store_dev(pa + dd, acc);
                else
                    *reinterpret_cast<float4v *>(pa + dd) = acc;
            }
            if (threadIdx.x % kDRuns == 0) {
                float *pm = a.part_ml + (size_t)(row0 + col) * a.ml_slot + slice * 2;
                if (a.merge > 0)
                    store_dev(pm, (float2){ms, lsum});
                else
                    *reinterpret_cast<float2 *>(pm) = (float2){ms, lsum};
            }
        }
    }
}

// ---- the splits merged by the workgroups themselves ---------------------------------------------------
// A plain launch of one sequence needs no second launch.  A workgroup that has written its partial takes
// a ticket of its group of kMergeGroup consecutive splits.  Whoever draws a group's last ticket finds every
// partial of the group in memory, folds them into one (in split order, so the result does not depend on
// who came last), writes that over the group's first partial and takes a ticket of the (item, KV head);
// whoever draws the last of those folds the groups' partials and writes the output rows, gated if the call
// says so.  Nobody waits for anybody: a workgroup that is not last leaves.  Two levels keep a fold at a few
// dozen KB (the 64 partials of a KV head with 6 heads are 384 KB, which one CU takes 3 us to read).
// The counters (`tickets`: per (item, KV head) one per group, then one for the groups) live in library
// memory, start at zero and are put back to zero by the workgroup that draws the last ticket, so a
// captured launch can be replayed; launches that share counters must not overlap.
constexpr int kMergeGroup = 8;
constexpr int kMergeMaxSplits = 128; // beyond: the merge kernels

// Thread 0 draws from `counter` once every thread's device-scope stores so far are visible to the device;
// returns (uniformly) whether this workgroup drew ticket `count` - 1: then every other drawer's stores are.
typedef volatile __attribute__((address_space(3))) unsigned int *LdsFlag;
__device__ __forceinline__ bool last_ticket(unsigned int *counter, unsigned int count, LdsFlag flag)
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // this thread's stores have been acknowledged
    __syncthreads(); // (also: everybody has read the flag of an earlier draw and is done with the LDS it lies in)
    if (threadIdx.x == 0) {
        const unsigned int drawn = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = drawn + 1 == count;
        if (last)
            __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = last ? 1u : 0u;
    }
    __syncthreads();
    return *flag != 0;
}

// (m, sum, KRUN values of d) of the partials first, first + step, ... (`count` of them) folded in that order:
// M = max m_j over the partials that saw a key (sum > 0), w_j = 2^(m_j - M), L = sum l_j w_j, A = sum acc_j w_j.
template <int KRUN>
__device__ __forceinline__ void fold_partials(const float *pa, const float *pm, int first, int step, int count,
                                              float &M, float &L, float4v (&A)[KRUN / 4])
{
    const float4v z = {0, 0, 0, 0};
    float2 v[8];
    float4v x[8][KRUN / 4];
    auto fetch = [&](int j0) {
#pragma unroll
        for (int jj = 0; jj < 8; jj++) {
            const int j = j0 + jj < count ? j0 + jj : count - 1; // (past the end: the last one again, weight 0)
            const size_t s = (size_t)first + (size_t)j * step;
            v[jj] = load_dev2(pm + s * 2);
#pragma unroll
            for (int i = 0; i < KRUN / 4; i++)
                x[jj][i] = load_dev4(pa + s * kHeadDim + 4 * i);
        }
    };
    fetch(0);
    M = -INFINITY;
#pragma unroll
    for (int jj = 0; jj < 8; jj++)
        M = jj < count && v[jj].y > 0.0f ? fmaxf(M, v[jj].x) : M;
    for (int j = 8; j < count; j++) {
        const float2 u = load_dev2(pm + ((size_t)first + (size_t)j * step) * 2);
        M = u.y > 0.0f ? fmaxf(M, u.x) : M;
    }
    L = 0.0f;
#pragma unroll
    for (int i = 0; i < KRUN / 4; i++)
        A[i] = z;
    for (int j0 = 0; j0 < count; j0 += 8) {
        if (j0 > 0)
            fetch(j0);
#pragma unroll
        for (int jj = 0; jj < 8; jj++) {
            const bool live = j0 + jj < count && v[jj].y > 0.0f; // (false for NaN as well)
            const float w = live ? __builtin_amdgcn_exp2f(v[jj].x - M) : 0.0f;
            L = fmaf(live ? v[jj].y : 0.0f, w, L);
            // a partial without a key holds whatever the scratch held: select, not multiply
#pragma unroll
            for (int i = 0; i < KRUN / 4; i++)
                A[i] += w > 0.0f ? x[jj][i] * w : z;
        }
    }
}

template <bool WIDE>
__device__ __forceinline__ void decode_merge_tail(const DecodeArgs &a, const Work &wk HIPML_STAMPS_ARG)
{
    constexpr int kCols = WIDE ? 16 : 8;
    constexpr int kDRuns = kThreads / kCols, kRun = kHeadDim / kDRuns; // as the partials were written
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_all[];
    const LdsFlag flag = (LdsFlag)lds_all;
    const int ngroup = (a.splits + kMergeGroup - 1) / kMergeGroup;
    const int g0 = wk.split / kMergeGroup * kMergeGroup;
    const int gsize = a.splits - g0 < kMergeGroup ? a.splits - g0 : kMergeGroup;
    unsigned int *tk = a.tickets + (size_t)(wk.item * a.n_kv + wk.kvh) * (ngroup + 1);
    const bool last1 = last_ticket(tk + g0 / kMergeGroup, (unsigned)gsize, flag);
    HIPML_STAMP(stamps_, 8); // the ticket of the group has come back
    if (!last1)
        return;
    const int nc = threadIdx.x / kDRuns;
    const int d0 = (threadIdx.x % kDRuns) * kRun;
    const bool mine = nc < wk.nvalid;
    const int col = mine ? nc / wk.group : 0;
    const int head = wk.hbase + (mine ? nc - col * wk.group : 0);
    float *pa = a.part_acc + (size_t)(wk.row0 + col) * a.acc_slot + (size_t)head * a.splits * kHeadDim + d0;
    float *pm = a.part_ml + (size_t)(wk.row0 + col) * a.ml_slot + (size_t)head * a.splits * 2;
    float M = -INFINITY, L = 0.0f;
    float4v A[kRun / 4];
    if (mine)
        fold_partials<kRun>(pa, pm, g0, 1, gsize, M, L, A);
    if (ngroup > 1) {
        if (mine) {
#pragma unroll
            for (int i = 0; i < kRun / 4; i++)
                store_dev(pa + (size_t)g0 * kHeadDim + 4 * i, A[i]);
            if (threadIdx.x % kDRuns == 0)
                store_dev(pm + (size_t)g0 * 2, (float2){M, L});
        }
        HIPML_STAMP(stamps_, 9); // the group's partials folded and stored
        const bool last2 = last_ticket(tk + ngroup, (unsigned)ngroup, flag);
        HIPML_STAMP(stamps_, 10); // the ticket of the KV head has come back
        if (!last2)
            return;
        if (mine)
            fold_partials<kRun>(pa, pm, 0, kMergeGroup, ngroup, M, L, A);
    }
    if (mine) {
        const size_t at = (size_t)(wk.row0 + col) * a.q_slot + (size_t)head * kHeadDim + d0;
        const float inv = L > 0.0f ? 1.0f / L : 0.0f;
#pragma unroll
        for (int i = 0; i < kRun / 4; i++) {
            float4v r = A[i] * inv;
            if (!(L > 0.0f))
                r = (float4v){0, 0, 0, 0};
            if (a.gate != nullptr) {
                const float4v gt = *reinterpret_cast<const float4v *>(a.gate + at + 4 * i);
                r = (float4v){gated(r[0], gt[0]), gated(r[1], gt[1]), gated(r[2], gt[2]), gated(r[3], gt[3])};
            }
            *reinterpret_cast<float4v *>(a.out + at + 4 * i) = r;
        }
    }
}

// One workgroup = one (KV head, key split, work item); the item's width picks the body.
// The kernel-argument segment of decode_q8_kernel, as the parameter list lays it out.
struct DecodeKernarg {
    const uint8_t *k, *v;
    const float *q;
    const int32_t *pos;
    int stride, splits;
    uint32_t wi, item0, geom, q_slot;
    DecodeArgs a;
};

__global__ void __launch_bounds__(kThreads, 2)
    decode_q8_kernel(const uint8_t *k, const uint8_t *v, const float *q, const int32_t *pos, int stride, int splits,
                     uint32_t wi, uint32_t item0, uint32_t geom, uint32_t q_slot, const DecodeArgs a)
{
    HIPML_STAMPS_DECL;
    HIPML_STAMP(stamps_, 0); // the wave's first instruction
    const Front f = front_of(k, v, q, pos, stride, splits, wi, item0, geom, q_slot, (uint32_t)offsetof(DecodeKernarg, a));
    Work wk;
    if (!find_work(a, f, threadIdx.x & 63, wk))
        return;
    HIPML_STAMP(stamps_, 1); // work item found
    if (wk.nvalid > 8) { // uniform over the workgroup
        decode_body_dma<true>(a, f, wk HIPML_STAMPS_PASS);
        HIPML_STAMP(stamps_, 7); // partial stored (not yet acknowledged)
        if (a.merge > 0)
            decode_merge_tail<true>(a, wk HIPML_STAMPS_PASS);
    } else {
        decode_body_dma<false>(a, f, wk HIPML_STAMPS_PASS);
        HIPML_STAMP(stamps_, 7);
        if (a.merge > 0)
            decode_merge_tail<false>(a, wk HIPML_STAMPS_PASS);
    }
#ifdef HIPML_DECODE_STAMPS
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    HIPML_STAMP(stamps_, 11); // everything this wave stored has been acknowledged
    stamps_out(stamps_);
#endif
}

// The same road for q4_0 rows (items of at most 8 columns: the launcher cuts wider slots by heads).
__global__ void __launch_bounds__(kThreads, 2)
    decode_q4_kernel(const uint8_t *k, const uint8_t *v, const float *q, const int32_t *pos, int stride, int splits,
                     uint32_t wi, uint32_t item0, uint32_t geom, uint32_t q_slot, const DecodeArgs a)
{
#ifdef HIPML_DECODE_STAMPS
    Stamps stamps_ = {}; // (not written out: the stamps are the q8_0 kernel's)
#endif
    const Front f = front_of(k, v, q, pos, stride, splits, wi, item0, geom, q_slot, (uint32_t)offsetof(DecodeKernarg, a));
    Work wk;
    if (!find_work(a, f, threadIdx.x & 63, wk))
        return;
    decode_body_dma<false, true>(a, f, wk HIPML_STAMPS_PASS);
}

// Wave-wide reductions without LDS: DPP inside a row of 16 lanes, then the two row-swap
// instructions (written as asm: the compiler's builtins for them return the first result twice).
template <bool MAX>
__device__ __forceinline__ float wave_reduce(float v)
{
    auto op = [](float a, float b) { return MAX ? fmaxf(a, b) : a + b; };
#define HIPML_DPP(x, ctrl)                                                                         \
    __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), ctrl, 0xf, \
                                                          0xf, true))
    v = op(v, HIPML_DPP(v, 0xB1));  // quad_perm [1,0,3,2]: lane ^ 1
    v = op(v, HIPML_DPP(v, 0x4E));  // quad_perm [2,3,0,1]: lane ^ 2
    v = op(v, HIPML_DPP(v, 0x141)); // row_half_mirror: the other quad of 8
    v = op(v, HIPML_DPP(v, 0x140)); // row_mirror: the other half of 16
#undef HIPML_DPP
    float a = v, b = v;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    v = op(a, b); // rows 0|1 and 2|3 combined
    a = v;
    b = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return op(a, b);
}

// out[row][head][d] = sum_s acc_s[d] * 2^(m_s - m) / sum_s l_s * 2^(m_s - m); 0 when no
// split saw a key.  grid (n_heads * 64 / (4 DL), rows): a workgroup owns 4 DL values of d of one
// (row, head); thread = (split group, float4 of d).  Latency matters more than bandwidth here:
// the first accumulator loads are issued before anything else, and the two reductions over
// the splits cost one barrier each.
constexpr int kReduceMaxSplits = 4096;

// DL = float4 lanes along d per workgroup (DL * 4 values), SG = 256 / DL split groups.
template <int DL>
__global__ void __launch_bounds__(256) decode_reduce_kernel(
    const float *__restrict__ part_acc, const float *__restrict__ part_ml, float *__restrict__ out,
    const float *__restrict__ gate, int splits, size_t acc_slot, size_t ml_slot, size_t q_slot)
{
    __shared__ float w_s[kReduceMaxSplits];
    __shared__ float red_m[4], red_l[4];
    constexpr int SG = 256 / DL;      // split groups
    constexpr int DQ = 64 / DL;       // workgroups per head
    __shared__ float4v accs[SG][DL];
    const int head = blockIdx.x / DQ;
    const int dq = blockIdx.x - head * DQ;
    const int row = blockIdx.y;
    const int tid = threadIdx.x;
    const int sg = tid / DL, dl = tid % DL;
    const float *ml = part_ml + (size_t)row * ml_slot + (size_t)head * splits * 2;
    const float *acc = part_acc + (size_t)row * acc_slot + (size_t)head * splits * kHeadDim +
                       dq * (DL * 4) + dl * 4;

    // first four accumulator rows of this thread, in flight while the weights are worked out
    float4v x0[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int s = sg + SG * k;
        x0[k] = (float4v){0, 0, 0, 0};
        if (s < splits)
            x0[k] = *reinterpret_cast<const float4v *>(acc + (size_t)s * kHeadDim);
    }
    // the output gate of the row (optional), fetched by the threads that write the result
    const size_t out_at = (size_t)row * q_slot + (size_t)head * kHeadDim + dq * (DL * 4) + (tid % DL) * 4;
    float4v gt = {0, 0, 0, 0};
    if (gate != nullptr && tid < DL)
        gt = *reinterpret_cast<const float4v *>(gate + out_at);

    // weights: w_s = 2^(m_s - m) for splits that saw a key, else 0
    float m = -INFINITY;
    for (int s = tid; s < splits; s += 256) {
        const float2 v = *reinterpret_cast<const float2 *>(ml + s * 2);
        if (v.y > 0.0f)
            m = fmaxf(m, v.x);
    }
    m = wave_reduce<true>(m);
    if ((tid & 63) == 0)
        red_m[tid >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red_m[0], red_m[1]), fmaxf(red_m[2], red_m[3]));
    float den = 0.0f;
    for (int s = tid; s < splits; s += 256) {
        const float2 v = *reinterpret_cast<const float2 *>(ml + s * 2); // L1 hit
        const float w = v.y > 0.0f ? __builtin_amdgcn_exp2f(v.x - m) : 0.0f;
        w_s[s] = w;
        den = fmaf(v.y > 0.0f ? v.y : 0.0f, w, den);
    }
    den = wave_reduce<false>(den);
    if ((tid & 63) == 0)
        red_l[tid >> 6] = den;
    __syncthreads();
    den = (red_l[0] + red_l[1]) + (red_l[2] + red_l[3]);

    float4v num = {0, 0, 0, 0};
    const float4v z = {0, 0, 0, 0};
    // zero-weight slices may hold anything (even NaN from an untouched scratch): select, not multiply
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int s = sg + SG * k;
        const float w = s < splits ? w_s[s] : 0.0f;
        num += w > 0.0f ? x0[k] * w : z;
    }
    auto term = [&](int s) {
        const float w = w_s[s];
        const float4v x = *reinterpret_cast<const float4v *>(acc + (size_t)s * kHeadDim);
        return w > 0.0f ? x * w : z;
    };
    int s = sg + 4 * SG;
    for (; s + 3 * SG < splits; s += 4 * SG)
        num += (term(s) + term(s + SG)) + (term(s + 2 * SG) + term(s + 3 * SG));
    for (; s < splits; s += SG)
        num += term(s);
    accs[sg][dl] = num;
    __syncthreads();
    if (tid < DL) {
        float4v t = accs[0][tid];
#pragma unroll
        for (int g = 1; g < SG; g++)
            t += accs[g][tid];
        const float inv = den > 0.0f ? 1.0f / den : 0.0f;
        float4v r = t * inv;
        if (!(den > 0.0f))
            r = (float4v){0, 0, 0, 0};
        if (gate != nullptr)
            r = (float4v){gated(r[0], gt[0]), gated(r[1], gt[1]), gated(r[2], gt[2]), gated(r[3], gt[3])};
        *reinterpret_cast<float4v *>(out + out_at) = r;
    }
}

// The same merge for at most 128 splits, with one barrier instead of three: every wave reads all
// (m, l) pairs of the (row, head) itself (lane j: splits 2j and 2j+1), so the maximum and the
// denominator are wave reductions without LDS, a thread takes the weights of its splits
// (sg + SG k) from the lanes that hold them, and the split groups of a wave meet through row
// rotations and the row-swap instructions; only the four waves' sums cross LDS.  Measured against
// the kernel above: 3.3 against 5.2 us for one row of 128 splits.
// grid (n_heads * 64 / (4 DL), rows), thread = (split group sg, float4 dl of d), as above.
// KN = splits per thread the launch needs (SG KN >= splits): the loops carry no run-time bounds.
template <int DL, int KN>
__global__ void __launch_bounds__(256) decode_reduce128_kernel(
    const float *__restrict__ part_acc, const float *__restrict__ part_ml, float *__restrict__ out,
    const float *__restrict__ gate, int splits, size_t acc_slot, size_t ml_slot, size_t q_slot)
{
    static_assert(DL == 4 || DL == 16, "split groups of a wave are reduced for 4 or 16 lanes of d");
    constexpr int SG = 256 / DL;   // split groups
    static_assert(KN >= 1 && SG * KN <= 128, "lane j of a wave holds the weights of splits 2j and 2j+1");
    constexpr int DQ = 64 / DL;    // workgroups per head
    __shared__ float4v accs[4][DL];
    const int head = blockIdx.x / DQ;
    const int dq = blockIdx.x - head * DQ;
    const int row = blockIdx.y;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int sg = tid / DL, dl = tid % DL;
    const float *ml = part_ml + (size_t)row * ml_slot + (size_t)head * splits * 2;
    const float *acc = part_acc + (size_t)row * acc_slot + (size_t)head * splits * kHeadDim +
                       dq * (DL * 4) + dl * 4;
    const float4v z = {0, 0, 0, 0};

    // the thread's accumulator rows first, then the wave's copy of the (m, l) table
    float4v x[KN];
#pragma unroll
    for (int k = 0; k < KN; k++) {
        // a split past the end repeats the last one (same cache line); its weight below is zero
        const int s = sg + SG * k < splits ? sg + SG * k : splits - 1;
        x[k] = *reinterpret_cast<const float4v *>(acc + (size_t)s * kHeadDim);
    }
    float2 v0 = {0.0f, 0.0f}, v1 = {0.0f, 0.0f};
    if (2 * lane < splits)
        v0 = *reinterpret_cast<const float2 *>(ml + 4 * lane);
    if (2 * lane + 1 < splits)
        v1 = *reinterpret_cast<const float2 *>(ml + 4 * lane + 2);
    const size_t out_at = (size_t)row * q_slot + (size_t)head * kHeadDim + dq * (DL * 4) + (tid % DL) * 4;
    float4v gt = z;
    if (gate != nullptr && tid < DL)
        gt = *reinterpret_cast<const float4v *>(gate + out_at);

    // weights: 2^(m_s - m) for splits that saw a key, else 0 (`l > 0` is false for NaN as well)
    const bool live0 = v0.y > 0.0f, live1 = v1.y > 0.0f;
    float m = fmaxf(live0 ? v0.x : -INFINITY, live1 ? v1.x : -INFINITY);
    m = wave_reduce<true>(m);
    const float w0 = live0 ? __builtin_amdgcn_exp2f(v0.x - m) : 0.0f;
    const float w1 = live1 ? __builtin_amdgcn_exp2f(v1.x - m) : 0.0f;
    float den = fmaf(live1 ? v1.y : 0.0f, w1, (live0 ? v0.y : 0.0f) * w0);
    den = wave_reduce<false>(den);
    // split s lives in lane s / 2, component s % 2 (SG is even: the component is that of sg)
    float4v num = z;
#pragma unroll
    for (int k = 0; k < KN; k++) {
        const int holder = ((sg >> 1) + (SG / 2) * k) * 4;
        const float c0 = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(holder, __builtin_bit_cast(int, w0)));
        const float c1 = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(holder, __builtin_bit_cast(int, w1)));
        const float w = (sg & 1) ? c1 : c0;
        // zero-weight slices may hold anything (even NaN from an untouched scratch): select, not multiply
        num += w > 0.0f ? x[k] * w : z;
    }
    // the split groups of the wave: lanes that differ in the bits above those of dl
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float v = num[j];
        if (DL == 4) {
            v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, true)); // row_ror:4
            v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, true)); // row_ror:8
        }
        num[j] = quad_rows<false>(v);
    }
    if (lane < DL)
        accs[wave][lane] = num;
    __syncthreads();
    if (tid < DL) {
        const float4v t = (accs[0][tid] + accs[1][tid]) + (accs[2][tid] + accs[3][tid]);
        const float inv = den > 0.0f ? 1.0f / den : 0.0f;
        float4v r = t * inv;
        if (!(den > 0.0f))
            r = z;
        if (gate != nullptr)
            r = (float4v){gated(r[0], gt[0]), gated(r[1], gt[1]), gated(r[2], gt[2]), gated(r[3], gt[3])};
        *reinterpret_cast<float4v *>(out + out_at) = r;
    }
}


int decode_init()
{
    struct { const void *fn; int bytes; } const kernels[] = {
        {reinterpret_cast<const void *>(&decode_q8_kernel), kDmaLds},
        {reinterpret_cast<const void *>(&decode_q4_kernel), kDmaLds},
        {reinterpret_cast<const void *>(&decode_staged_kernel<false, true>), decode_lds_bytes(1)},
        {reinterpret_cast<const void *>(&decode_staged_kernel<true, false>), decode_lds_bytes(1)},
    };
    for (const auto &k : kernels) {
        const hipError_t e = hipFuncSetAttribute(k.fn, hipFuncAttributeMaxDynamicSharedMemorySize, k.bytes);
        if (e != hipSuccess)
            return fail((int)e, "hipFuncSetAttribute(decode LDS) failed: %d (%s)", (int)e, hipGetErrorString(e));
    }
    return 0;
}

// ---- partials without an allocation -------------------------------------------------------------
// hipml_attn_decode_kv_noalloc keeps the split partials of a call in this array instead of in buffers
// the caller brings: every GPU the library is initialised on holds one copy (4,227,072 bytes) until
// the process ends.  In host code the name `scratch` is only a handle for the symbol; the memory is
// reached through the address hipGetSymbolAddress returns for the current device, kept per device.
constexpr size_t kStaticSlices = 4096; // (head, split) pairs: n_heads * splits of a call
static __device__ __align__(256) float scratch[kStaticSlices * (kHeadDim + 2)];
constexpr int kMaxDevices = 64;
static std::atomic<float *> g_scratch_ptr[kMaxDevices]; // device address of `scratch` on each initialised GPU

static int decode_tickets_init(int device);

// Called by hipml_attn_init with `device` current.
int decode_static_init(int device)
{
    if (device < 0 || device >= kMaxDevices)
        return fail(HIPML_ATTN_E_RANGE, "device %d outside 0..%d", device, kMaxDevices - 1);
    float *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
        return fail(e != hipSuccess ? (int)e : HIPML_ATTN_E_STATE, "hipGetSymbolAddress(scratch) failed: %d (%s)",
                    (int)e, hipGetErrorString(e));
    g_scratch_ptr[device] = ptr;
    return decode_tickets_init(device);
}

// ---- arrival counters of the launches whose workgroups merge their own partials ---------------------
// (decode_merge_tail).  Launches that may run at the same time need counters of their own, and launches
// on one stream never do, so a launch takes the slot of its stream: the first kTicketStreams streams a
// device sees get one each, for good; launches on further streams go the way of two launches.  A launch
// that is being captured into a graph takes the next slot of a ring instead, because a graph may be
// replayed on any stream and beside eager launches of the stream it was captured on: two graphs whose
// captured launches are kTicketRing launches apart share slots and must not be replayed at the same time.
// Every GPU the library is initialised on holds one copy of the array (512 KiB), zero when the module is
// loaded; a kernel leaves the counters it used at zero.
// Whether they do is a setting of the process, off unless asked for: measured on MI355X the device-scope
// round trips of one level of this merge (stores acknowledged, ticket, loads: ~1.2 us each) cost as much as
// the launch of the merge kernel they replace, so the two launches are the faster form at every depth.
static std::atomic<int> g_one_launch{[] {
    const char *e = getenv("HIPML_DECODE_ONE_LAUNCH");
    return e != nullptr && e[0] != '\0' && e[0] != '0' ? 1 : 0;
}()};
int decode_one_launch(int on)
{
    return on < 0 ? g_one_launch.load(std::memory_order_relaxed) : g_one_launch.exchange(on != 0 ? 1 : 0);
}

constexpr int kTicketStreams = 32, kTicketRing = 96;
constexpr int kTicketsPerSlot = 1024;
static __device__ __align__(256) unsigned int tickets[(kTicketStreams + kTicketRing) * kTicketsPerSlot];
static unsigned int *g_tickets_ptr[kMaxDevices];
static std::mutex g_ticket_mu;
static hipStream_t g_ticket_stream[kMaxDevices][kTicketStreams];
static int g_ticket_streams[kMaxDevices];
static unsigned int g_ticket_ring[kMaxDevices];

static int decode_tickets_init(int device)
{
    unsigned int *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(tickets));
    if (e != hipSuccess || ptr == nullptr)
        return fail(e != hipSuccess ? (int)e : HIPML_ATTN_E_STATE, "hipGetSymbolAddress(tickets) failed: %d (%s)",
                    (int)e, hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(g_ticket_mu);
    g_tickets_ptr[device] = ptr;
    return 0;
}

// The counters a launch of `need` of them on `st` may use, or nullptr: then the launch leaves the merge
// to a second one.  Allocates nothing and launches nothing.
static unsigned int *decode_tickets(hipStream_t st, int need)
{
    if (g_one_launch.load(std::memory_order_relaxed) == 0 || need > kTicketsPerSlot)
        return nullptr;
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices)
        return nullptr;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &capture) != hipSuccess) {
        (void)hipGetLastError(); // (the launch itself will report what is wrong with the stream)
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_ticket_mu);
    unsigned int *base = g_tickets_ptr[device];
    if (base == nullptr)
        return nullptr;
    if (capture != hipStreamCaptureStatusNone)
        return base + (size_t)(kTicketStreams + g_ticket_ring[device]++ % kTicketRing) * kTicketsPerSlot;
    int n = g_ticket_streams[device], i = 0;
    while (i < n && g_ticket_stream[device][i] != st)
        i++;
    if (i == n) {
        if (n == kTicketStreams)
            return nullptr;
        g_ticket_stream[device][n] = st;
        g_ticket_streams[device] = n + 1;
    }
    return base + (size_t)i * kTicketsPerSlot;
}

// The current device's copy of the array, cut into the two partial buffers of a decode call of
// n_heads x splits slices; nothing is allocated.
int decode_static_partials(int n_heads, int splits, float **part_acc, float **part_ml)
{
    int device = -1;
    const hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess)
        return fail((int)e, "hipGetDevice failed: %d (%s)", (int)e, hipGetErrorString(e));
    if (device < 0 || device >= kMaxDevices || g_scratch_ptr[device].load() == nullptr)
        return fail(HIPML_ATTN_E_STATE, "hipml_attn_init has not been called for device %d", device);
    if (n_heads < 1 || splits < 1 || (size_t)n_heads * (size_t)splits > kStaticSlices)
        return fail(HIPML_ATTN_E_RANGE,
                    "n_heads %d x splits %d: the built-in scratch holds at most %zu (head, split) partials",
                    n_heads, splits, kStaticSlices);
    float *ptr = g_scratch_ptr[device].load();
    *part_acc = ptr;
    *part_ml = ptr + (size_t)n_heads * (size_t)splits * kHeadDim;
    return 0;
}

// ---- head widths other than 256 ------------------------------------------------------------------------
// The reference's decode launchers take any head_dim that is a multiple of the block size, and its
// parity table runs head_dim 64 (crates/hipml-core/src/parity_kv.rs:166-213).  The model this library
// is built for has head_dim 256 and every kernel above is laid out for that; the two kernels below serve
// head_dim 64 with the same arguments, partial format and merge rule, in plain fp32 arithmetic: one wave
// per (query row, head, key split), one key per lane and turn, the lane's running maximum, sum and
// head_dim accumulators in registers, the lanes' states merged with lane exchanges at the end.  They are
// there for completeness of the interface, not tuned.
struct DecodeHdArgs {
    const float *q;
    const uint8_t *k;
    const uint8_t *v;
    float *part_acc;
    float *part_ml;
    float *out;
    const float *gate;
    const int32_t *pos;
    int n_heads, n_kv, group, stride, splits;
    float scale_log2; // scale * log2(e)
    size_t kv_slot_bytes, acc_slot, ml_slot, q_slot;
    uint8_t slot_of_row[kMaxSlots * kMaxCols];
};

// block b of a cached row as 32 floats (f16 scale x integer)
template <bool Q4>
__device__ __forceinline__ void hd_block(const uint8_t *row, int b, float (&x)[32])
{
    constexpr int kBlockBytes = Q4 ? kQ4BlockBytes : kQ8BlockBytes;
    const uint16_t *w = reinterpret_cast<const uint16_t *>(row + b * kBlockBytes); // blocks are 2-byte aligned
    const float d = (float)__builtin_bit_cast(_Float16, w[0]);
    if (Q4) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t two = w[1 + j]; // bytes 2j, 2j + 1: elements 2j, 2j + 1 in the low nibbles, + 16 in the high ones
            x[2 * j] = d * (float)((int)(two & 15) - 8);
            x[2 * j + 16] = d * (float)((int)((two >> 4) & 15) - 8);
            x[2 * j + 1] = d * (float)((int)((two >> 8) & 15) - 8);
            x[2 * j + 17] = d * (float)((int)((two >> 12) & 15) - 8);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const uint32_t two = w[1 + j];
            x[2 * j] = d * (float)(int8_t)(two & 0xff);
            x[2 * j + 1] = d * (float)(int8_t)(two >> 8);
        }
    }
}

template <int HD, bool Q4>
__global__ void __launch_bounds__(64 * kMaxGroup, 1) decode_hd_kernel(const DecodeHdArgs a)
{
    constexpr int kRow = HD / 32 * (Q4 ? kQ4BlockBytes : kQ8BlockBytes);
    __shared__ float qs[kMaxGroup][HD];
    const int lane = threadIdx.x & 63, hq = threadIdx.x >> 6;
    const int kvh = blockIdx.x / a.splits, split = blockIdx.x - kvh * a.splits;
    const int r = blockIdx.y;
    const int head = kvh * a.group + hq;
    for (int d = lane; d < HD; d += 64)
        qs[hq][d] = a.q[(size_t)r * a.q_slot + (size_t)head * HD + d];
    __syncthreads();
    int seq = a.pos[2 * r + 1];
    seq = seq < 0 ? 0 : (seq > a.stride ? a.stride : seq);
    const int per = (seq + a.splits - 1) / a.splits; // the reference's partition (attn_decode_kv_w.hip:124-126)
    const int lo = split * per;
    const int hi = lo + per < seq ? lo + per : seq;
    const size_t base = (size_t)a.slot_of_row[r] * a.kv_slot_bytes + (size_t)kvh * a.stride * kRow;
    float m = -INFINITY, l = 0.0f, acc[HD];
#pragma unroll
    for (int d = 0; d < HD; d++)
        acc[d] = 0.0f;
    for (int key = lo + lane; key < hi; key += 64) {
        float x[32];
        float dot = 0.0f;
#pragma unroll
        for (int b = 0; b < HD / 32; b++) {
            hd_block<Q4>(a.k + base + (size_t)key * kRow, b, x);
#pragma unroll
            for (int d = 0; d < 32; d++)
                dot = fmaf(qs[hq][b * 32 + d], x[d], dot);
        }
        const float sc = dot * a.scale_log2;
        const float mn = fmaxf(m, sc);
        const float corr = __builtin_amdgcn_exp2f(m - mn); // (m = -inf the first time: 0)
        const float pr = __builtin_amdgcn_exp2f(sc - mn);
        l = l * corr + pr;
#pragma unroll
        for (int b = 0; b < HD / 32; b++) {
            hd_block<Q4>(a.v + base + (size_t)key * kRow, b, x);
#pragma unroll
            for (int d = 0; d < 32; d++)
                acc[b * 32 + d] = fmaf(pr, x[d], acc[b * 32 + d] * corr);
        }
        m = mn;
    }
    // the lanes' states against the wave's maximum
    float mw = m;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        mw = fmaxf(mw, __shfl_xor(mw, o));
    const float w = m == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m - mw);
    float lw = l * w;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        lw += __shfl_xor(lw, o);
    const size_t part = (size_t)head * a.splits + split;
    float *pa = a.part_acc + (size_t)r * a.acc_slot + part * HD;
#pragma unroll
    for (int d = 0; d < HD; d++) {
        float t = acc[d] * w;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1)
            t += __shfl_xor(t, o);
        if (lane == (d & 63))
            pa[d] = t;
    }
    if (lane == 0) {
        float *pm = a.part_ml + (size_t)r * a.ml_slot + part * 2;
        pm[0] = lw > 0.0f ? mw : 0.0f;
        pm[1] = lw;
    }
}

// out[row][head][d] = sum_s acc_s[d] 2^(m_s - m) / sum_s l_s 2^(m_s - m), 0 when no split saw a key
// (crates/hipml-kernels/kernels/attn_decode_kv.hip:491-532); grid (n_heads, rows), one thread per d.
template <int HD>
__global__ void __launch_bounds__(HD) decode_hd_reduce_kernel(const DecodeHdArgs a)
{
    const int head = blockIdx.x, r = blockIdx.y, d = threadIdx.x;
    const float *pm = a.part_ml + (size_t)r * a.ml_slot + (size_t)head * a.splits * 2;
    const float *pa = a.part_acc + (size_t)r * a.acc_slot + (size_t)head * a.splits * HD;
    float m = -INFINITY;
    for (int s = 0; s < a.splits; s++)
        if (pm[2 * s + 1] > 0.0f)
            m = fmaxf(m, pm[2 * s]);
    float num = 0.0f, den = 0.0f;
    for (int s = 0; s < a.splits; s++) {
        const float ls = pm[2 * s + 1];
        if (ls > 0.0f) {
            const float w = __builtin_amdgcn_exp2f(pm[2 * s] - m);
            num = fmaf(pa[(size_t)s * HD + d], w, num);
            den = fmaf(ls, w, den);
        }
    }
    float y = den > 0.0f ? num / den : 0.0f;
    const size_t at = (size_t)r * a.q_slot + (size_t)head * HD + d;
    if (a.gate)
        y = gated(y, a.gate[at]);
    a.out[at] = y;
}

static int launch_decode_hd(hipStream_t st, const DecodeLaunch &L)
{
    DecodeHdArgs a;
    a.q = L.q;
    a.k = L.k;
    a.v = L.v;
    a.part_acc = L.part_acc;
    a.part_ml = L.part_ml;
    a.out = L.out;
    a.gate = L.gate;
    a.pos = L.pos;
    a.n_heads = L.n_heads;
    a.n_kv = L.n_kv;
    a.group = L.n_heads / L.n_kv;
    a.stride = L.stride;
    a.splits = L.splits;
    a.scale_log2 = L.scale * kLog2e;
    a.kv_slot_bytes = L.kv_slot_bytes;
    a.acc_slot = L.acc_slot;
    a.ml_slot = L.ml_slot;
    a.q_slot = L.q_slot;
    memset(a.slot_of_row, 0, sizeof(a.slot_of_row));
    for (int s = 0; s < L.slots; s++)
        for (int c = 0; c < L.cols[s]; c++)
            a.slot_of_row[L.row0[s] + c] = (uint8_t)s;
    const dim3 grid((unsigned)(L.n_kv * L.splits), (unsigned)L.total_rows, 1), block((unsigned)(64 * a.group), 1, 1);
    const dim3 rgrid((unsigned)L.n_heads, (unsigned)L.total_rows, 1);
    if (L.head_dim != 64)
        return fail(HIPML_ATTN_E_SHAPE, "head_dim %d: 256 and 64 are built", L.head_dim);
    if (L.q4)
        HIPML_LAUNCH((decode_hd_kernel<64, true>), grid, block, 0, st, a);
    else
        HIPML_LAUNCH((decode_hd_kernel<64, false>), grid, block, 0, st, a);
    int rc = launched("attn_decode_kv_hd");
    if (rc)
        return rc;
    HIPML_LAUNCH(decode_hd_reduce_kernel<64>, rgrid, dim3(64, 1, 1), 0, st, a);
    return launched("attn_decode_kv_hd_reduce");
}

int launch_decode_q8(hipStream_t st, const DecodeLaunch &given)
{
    if (given.head_dim != kHeadDim)
        return launch_decode_hd(st, given);
    DecodeLaunch L = given;
    // q8_0 and q4_0: the kernel that streams raw rows into LDS (it addresses a KV head's rows and the Q rows
    // with 32-bit byte offsets); the fp32-class variant and caches of more than 4 GiB per KV head: the staged
    // kernel
    const bool raw_rows = !L.exact && (size_t)L.stride * kRowBytes < ((size_t)1 << 32) &&
                          ((size_t)L.total_rows * L.q_slot + (size_t)L.n_heads * kHeadDim) * sizeof(float) <
                              ((size_t)1 << 32);
    // One sequence over q8_0: the raw-row kernel is at its best with one workgroup per CU (19.2 us per layer at
    // depth 32,768 with 64 splits of 4 KV heads, 20.4 with 128).  Over q4_0 a workgroup has half the bytes to
    // wait for and more arithmetic per byte, and two per CU pay from about 24,000 rows on (one / two per CU:
    // 10.4 / 11.5 us at 8,192, 16.5 / 16.2 at 32,768, 44.1 / 36.1 at 131,072).  The split policy sizes the
    // scratch for two; a launch that runs one per CU cuts the keys into half as many splits and leaves the rest
    // of the scratch alone (the layout of the partials is the kernels' own; every row of a verify group is cut
    // the same way as its plain decode).
    if (raw_rows && L.slots == 1 && !(L.q4 && L.stride >= 24576)) {
        const int one_per_cu = 256 / L.n_kv > 1 ? 256 / L.n_kv : 1;
        L.splits = L.splits < one_per_cu ? L.splits : one_per_cu;
    }
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
    memset(a.row0, 0, sizeof(a.row0));
    memset(a.cols, 0, sizeof(a.cols));
    memset(a.kvslot, 0, sizeof(a.kvslot));
    memset(a.head0, 0, sizeof(a.head0));
    memset(a.nhead, 0, sizeof(a.nhead));
    // Work items: a slot whose rows x heads fit 8 columns is one item; a wider one (rows of an
    // MTP-verify slot) is cut by heads into as few items of at most 16 columns as will do, of equal
    // width where the heads divide that way (3 rows x 6 heads: two items of 9 columns).
    int items = 0;
    for (int s = 0; s < L.slots; s++) {
        const int cols = L.cols[s];
        // (the raw-row kernel runs items of up to 8 columns through its narrow body and, over q8_0, wider ones
        // through its wide one; over q4_0 every item has at most 8)
        const int cap = raw_rows && L.q4 ? 8 : (!raw_rows || cols * a.group > 8 ? 16 : 8);
        const int per_max = cap / cols;                           // heads per item: 2..16 (cols <= 4)
        const int n_items = (a.group + per_max - 1) / per_max;
        const int base = a.group / n_items, extra = a.group % n_items;
        for (int i = 0, h0 = 0; i < n_items; i++) {
            const int nh = base + (i < extra ? 1 : 0);
            a.row0[items] = L.row0[s];
            a.cols[items] = (uint8_t)cols;
            a.kvslot[items] = (uint8_t)s;
            a.head0[items] = (uint8_t)h0;
            a.nhead[items] = (uint8_t)nh;
            h0 += nh;
            items++;
        }
    }
    a.items = items;
    a.stream_once = items == 1;
    a.i0_row0 = a.row0[0];
    a.i0_cols = a.cols[0];
    a.i0_slot = a.kvslot[0];
    a.i0_head0 = a.head0[0];
    a.i0_nhead = a.nhead[0];
    // batches: one window of workers (two workgroups per CU over 256 CUs), as long as every item can
    // have a worker of its own and lane i of a wave can look at item i
    // (the items of one sequence, a verify group, share their depth: the plain grid gives every row
    // the tile-to-split partition its plain decode has, so that its result is the same bit for bit)
    const int window = 512 / L.n_kv;
    a.workers = L.slots > 1 && items > 1 && items <= 64 && 2 * items <= window ? window : 0;
    const dim3 grid = a.workers > 0 ? dim3((unsigned)(L.n_kv * a.workers), 1, 1)
                                    : dim3((unsigned)(L.n_kv * L.splits), (unsigned)items, 1);
    // One sequence over q8_0 rows: the workgroups merge their partials themselves, if this stream has
    // counters for them (one row and the rows of a verify group alike, so that a column of a group stays
    // bit for bit the plain decode of its row).
    a.out = L.out;
    a.gate = L.gate;
    a.tickets = nullptr;
    a.merge = 0;
    if (raw_rows && !L.q4 && L.slots == 1 && a.workers == 0 && L.splits <= kMergeMaxSplits) {
        const int ngroup = (L.splits + kMergeGroup - 1) / kMergeGroup;
        a.tickets = decode_tickets(st, items * L.n_kv * (ngroup + 1));
        a.merge = a.tickets != nullptr ? kMergeGroup : 0;
    }
    if (raw_rows) {
        // the leading arguments (see Front): a launch with one item gets its caches at that item's slot
        const size_t slot_at = items == 1 ? (size_t)a.i0_slot * a.kv_slot_bytes : 0;
        const uint32_t wi = (uint32_t)a.workers | (uint32_t)items << 16;
        const uint32_t item0 = (uint32_t)a.i0_row0 | (uint32_t)a.i0_cols << 10 | (uint32_t)a.i0_head0 << 13 |
                               (uint32_t)a.i0_nhead << 16 | (uint32_t)a.i0_slot << 20;
        const uint32_t geom = (uint32_t)a.group | (uint32_t)a.n_kv << 4 | (uint32_t)a.stream_once << 20;
        if (L.q4)
            HIPML_LAUNCH(decode_q4_kernel, grid, dim3(kThreads, 1, 1), kDmaLds, st, a.k + slot_at, a.v + slot_at, a.q,
                         a.pos, a.stride, a.splits, wi, item0, geom, (uint32_t)a.q_slot, a);
        else
            HIPML_LAUNCH(decode_q8_kernel, grid, dim3(kThreads, 1, 1), kDmaLds, st, a.k + slot_at, a.v + slot_at, a.q,
                         a.pos, a.stride, a.splits, wi, item0, geom, (uint32_t)a.q_slot, a);
    }
    else if (L.q4)
        HIPML_LAUNCH((decode_staged_kernel<true, false>), grid, dim3(kThreads, 1, 1), decode_lds_bytes(1), st, a);
    else
        HIPML_LAUNCH((decode_staged_kernel<false, true>), grid, dim3(kThreads, 1, 1), decode_lds_bytes(1), st, a);
    int rc = launched(L.q4 ? "attn_decode_kv_q4" : "attn_decode_kv_q8");
    if (rc || a.merge > 0)
        return rc;
    // Up to 128 splits (every launch the split policies make): the one-barrier merge.  One sequence
    // (a query row, or the rows of a verify group: the same merge, so that a column of a group is
    // bit for bit the plain decode of its row, as the reference's column check demands): 16 d per
    // workgroup (four times the workgroups, 64-byte pieces of a partial row per thread group);
    // a batch: 64 d per workgroup.
    if (L.splits <= 128 && L.slots == 1) {
        const dim3 grid((unsigned)L.n_heads * 16, (unsigned)L.total_rows, 1);
        if (L.splits <= 64)
            HIPML_LAUNCH((decode_reduce128_kernel<4, 1>), grid, dim3(256, 1, 1), 0, st, L.part_acc, L.part_ml,
                               L.out, L.gate, L.splits, L.acc_slot, L.ml_slot, L.q_slot);
        else
            HIPML_LAUNCH((decode_reduce128_kernel<4, 2>), grid, dim3(256, 1, 1), 0, st, L.part_acc, L.part_ml,
                               L.out, L.gate, L.splits, L.acc_slot, L.ml_slot, L.q_slot);
    } else if (L.splits <= 128) {
        const dim3 grid((unsigned)L.n_heads * 4, (unsigned)L.total_rows, 1);
        if (L.splits <= 16)
            HIPML_LAUNCH((decode_reduce128_kernel<16, 1>), grid, dim3(256, 1, 1), 0, st, L.part_acc, L.part_ml,
                               L.out, L.gate, L.splits, L.acc_slot, L.ml_slot, L.q_slot);
        else if (L.splits <= 32)
            HIPML_LAUNCH((decode_reduce128_kernel<16, 2>), grid, dim3(256, 1, 1), 0, st, L.part_acc, L.part_ml,
                               L.out, L.gate, L.splits, L.acc_slot, L.ml_slot, L.q_slot);
        else if (L.splits <= 64)
            HIPML_LAUNCH((decode_reduce128_kernel<16, 4>), grid, dim3(256, 1, 1), 0, st, L.part_acc, L.part_ml,
                               L.out, L.gate, L.splits, L.acc_slot, L.ml_slot, L.q_slot);
        else
            HIPML_LAUNCH((decode_reduce128_kernel<16, 8>), grid, dim3(256, 1, 1), 0, st, L.part_acc, L.part_ml,
                               L.out, L.gate, L.splits, L.acc_slot, L.ml_slot, L.q_slot);
    }
    else if (L.slots == 1)
        HIPML_LAUNCH(decode_reduce_kernel<4>, dim3((unsigned)L.n_heads * 16, (unsigned)L.total_rows, 1), dim3(256, 1, 1), 0,
                           st, L.part_acc, L.part_ml, L.out, L.gate, L.splits, L.acc_slot, L.ml_slot, L.q_slot);
    else
        HIPML_LAUNCH(decode_reduce_kernel<16>,
                           dim3((unsigned)L.n_heads * 4, (unsigned)L.total_rows, 1), dim3(256, 1, 1), 0,
                           st, L.part_acc, L.part_ml, L.out, L.gate, L.splits, L.acc_slot, L.ml_slot, L.q_slot);
    return launched("attn_decode_kv_reduce");
}

} // namespace hipml

#ifdef HIPML_DECODE_STAMPS
// Instrumented builds only: the stamps of the most recent decode_q8_kernel launch, [workgroup][12] ticks of the
// 100 MHz counter (0 where a workgroup did not pass a point); returns a hipError_t.
extern "C" int hipml_dbg_decode_stamps(unsigned long long *host, size_t n) { return hipml::decode_read_stamps(host, n); }
#endif
