/*
 * hipml_attn.h -- C ABI of libhipml_attn.so: the full-attention hot path of the
 * qwen35 hybrid (RoPE, q8_0 KV append, split-K decode, MTP-verify decode,
 * batched decode, causal GQA chunk prefill, sigmoid output gate) for MI355X
 * (gfx950).  One entry point per launcher of the reference's kernel crate; the
 * citation on each prototype is the reference function it replaces
 * (paths relative to the reference repository).
 *
 * Conventions shared by every entry point
 *   - All pointers are device pointers unless the name says `host`.
 *   - `stream` is a hipStream_t passed as void*.  Launches are asynchronous on
 *     it; nothing here synchronises, allocates or frees, so every call is legal
 *     under stream capture.  Per-step scalars (position, live length) are read
 *     from device memory exactly as the reference's kernels do.
 *   - Return value: 0 on success; a negative hipml_attn_status for an argument
 *     error detected before any launch; a positive hipError_t if the runtime
 *     refused the launch.  hipml_attn_last_error() returns a thread-local
 *     message for the last non-zero return.
 *   - Layouts: Q / out / gate are f32 [rows][n_heads][head_dim].  A q8_0 cache
 *     is two byte arrays K and V of [n_kv][stride][head_dim/32] 34-byte blocks
 *     (f16 scale, 32 x int8): block (kvh,pos,c) starts at byte
 *     ((kvh*stride + pos)*(head_dim/32) + c)*34      (crates/hipml-core/src/kv.rs:22-40).
 *     A q4_0 cache has the same shape with 18-byte blocks (f16 scale, 16 bytes whose low /
 *     high nibbles are elements j / j+16; value = (nibble - 8) * scale, kv.rs:201-218).
 *   - `dtype` of the append entry points is the reference's KvDtype id: 0 = q8_0, 1 = q4_0.
 *     The decode entry points take the reference's kernel selector: 0 or 4 = q8_0, 1 or 5 =
 *     q4_0, 6 = q8_0 through the fp32-class kernel (in the reference 6 keeps its staged q8_0
 *     kernel reachable next to the shipped one; here it selects the variant that carries the
 *     softmax weights as hi + lo f16 pairs and meets the reference's 1e-4 / 1e-3 parity
 *     tolerance, at a lower speed) (crates/hipml-kernels/src/launch_kv.rs:146-170,329-334;
 *     its other values pick variants of the reference's own kernels and are rejected).  The
 *     chunk entry points
 *     take 1 = q8_0, 2 = q4_0 (attn_gpu/imp/attn_chunk_kv.rs:41-60).
 */
#ifndef HIPML_ATTN_H
#define HIPML_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *hipml_stream_t; /* hipStream_t */

typedef enum hipml_attn_status {
    HIPML_ATTN_OK = 0,
    HIPML_ATTN_E_SHAPE = -1,       /* head counts / head_dim / group the kernels do not cover */
    HIPML_ATTN_E_UNSUPPORTED = -2, /* unknown or unsupported dtype / variant */
    HIPML_ATTN_E_NULL = -3,        /* a required pointer is NULL */
    HIPML_ATTN_E_RANGE = -4,       /* a count or offset is out of range */
    HIPML_ATTN_E_DEVICE = -5,      /* not a gfx950 device */
    HIPML_ATTN_E_STATE = -6        /* required set-up call missing (e.g. no RoPE table) */
} hipml_attn_status;

/* ---- library ------------------------------------------------------------ */

/* Prepare `device`: check that it is gfx950, raise the kernels' LDS limits and look up the
 * library's built-in scratch array there.  The caller's current device is left as it was;
 * launches go to whatever device is current at the call and need this set-up for that device
 * (HIPML_ATTN_E_STATE otherwise).  Replaces Launcher::new's module load,
 * crates/hipml-kernels/src/launch.rs:119-141. */
int hipml_attn_init(int device);
/* Thread-local text for the last failure on this thread ("" if none). */
const char *hipml_attn_last_error(void);
const char *hipml_attn_version(void);

/* ---- split policies (host arithmetic, no GPU) ----------------------------
 * The three policies are tuned for the chip and the model this library is built for and say so nowhere in
 * their arguments: 256 CUs in 8 XCDs (one or two workgroups per CU, windows of 256 or 512 workgroups), and 6
 * query heads per KV head wherever a count depends on the heads (the chunk policies size task blocks and
 * the tiles' room in the scratch for 6).  Other head groupings work with the counts they return; they are
 * merely not the measured optimum there. */

/* Key splits for single-sequence decode on MI355X.  Same role as
 * DeepKv::splits, crates/hipml-model/src/gpu/deep_kv.rs:102-110, retuned for
 * 256 CUs.  Scratch is [n_heads][splits][head_dim] + [n_heads][splits][2] f32.  The count is what the q4_0
 * kernel wants (two workgroups per CU); over q8_0 a single-sequence launch given more than 256 / n_kv splits
 * runs that many (one workgroup per CU, its optimum) inside the same scratch. */
int hipml_attn_decode_splits(int seq, int n_kv);
/* Key splits for batched decode.  Same role as attn_splits,
 * crates/hipml-model/src/gpu/batch/kv.rs:39-42. */
int hipml_attn_batch_splits(int stride, int n_kv, int slots);
/* Key splits for a prefill chunk starting at pos0.  Same role as split_count,
 * crates/hipml-model/src/gpu/attn_tile.rs:138-151.  0 (chunks near position 0: pos0 + tokens <=
 * 1,792 and pos0 <= 2 * tokens) selects the kernel that cuts the keys inside its workgroups and
 * needs no scratch; 1 the single-pass kernel; n >= 2 that kernel over n key slices with scratch
 * and a merge launch.  For long chunks behind a prefix at least as long (tokens >= 768 and pos0 >= tokens, or tokens >= 640
 * and pos0 >= 8 * tokens) n is larger
 * than the number of slices that run (hipml_attn_chunk_slices): the chunk entry points then write the
 * live rows of the cache as f16 tiles (70,656 bytes per KV head and 64 rows) into the tail of part_acc
 * and run the attention over those, which is faster than dequantizing inside the attention (2,048 tokens
 * at depth 100,000: n = 13 for 4 slices, 654 MB of scratch, 4.1 against 4.7 ms).  A caller that passes a
 * smaller n (the reference's own policy gives 8) gets n slices of the kernel that dequantizes for itself:
 * the scratch is never written beyond the n slices it was sized for.
 * How that count grows: the partial rows are ceil32(tokens) * n_heads * 1,024 bytes per slice (50.3 MB at
 * 2,048 tokens and 24 heads), the tiles n_kv * ceil((pos0 + tokens) / 64) * 70,656 bytes (4.4 MB per 1,000
 * rows of depth at 4 KV heads), so n = slices + ceil(tiles / partial rows of one slice): 2,048-token chunks
 * at depth 32,768 / 100,000 / 200,000 / 400,000: 8 / 13 / 22 / 40, i.e. 0.40 / 0.65 / 1.1 / 2.0 GB.  The
 * reference caps its scratch at 1 GiB (crates/hipml-model/src/gpu/prefill.rs:159-166); an engine that keeps
 * that cap passes the count its allocation holds, and from ~195,000 positions on that is the kernel that
 * dequantizes for itself again.  Counts above 64 are never returned (the plain slice count is, instead).
 * An engine that registers its caches with hipml_kv_f16_attach needs none of this: the tiles then live
 * in the cache's own shadow, the count only has to cover the slices that run (hipml_attn_chunk_slices:
 * 4 at these shapes), and 8 is always enough.
 * NOTE: unlike the reference's split_count, which is at least 1, this returns 0 near position 0. */
int hipml_attn_chunk_splits(int pos0, int tokens, int n_kv);
/* The slice count (>= 1) for callers that want the sliced kernel whatever the shape, and for
 * hipml_attn_chunk_kv_f16, which has no in-workgroup variant: what hipml_attn_chunk_splits
 * returns where it does not return 0. */
int hipml_attn_chunk_slices(int pos0, int tokens, int n_kv);

/* ---- RoPE ----------------------------------------------------------------
 * The reference's CPU definition builds the angle in f64 with the host libm
 * (crates/hipml-core/src/ops.rs:296-305).  To be bit-identical to it the
 * kernels read cos/sin from a table the HOST fills with that same libm:
 * table[pos][k] = { (float)cos(pos * theta^(-2k/n_rot)), (float)sin(...) },
 * f32 [max_pos][n_rot/2][2]. */
size_t hipml_rope_table_bytes(int n_rot, int max_pos);
int hipml_rope_table_fill_host(float *host_table, float theta_base, int n_rot, int max_pos);
/* Register a device copy of the table (caller owns the memory; the engine registers n_ctx rows).
 * The table and the switch below belong to the device that is current when they are set (the pointer is
 * that device's memory), one registration per device; they may be set from any thread, and a call that
 * is already running keeps the registration it started with.  Without a table for (theta_base, n_rot) on
 * the current device the RoPE entry points return
 * HIPML_ATTN_E_STATE.  A position at or beyond max_pos is an error: HIPML_ATTN_E_RANGE where the
 * host knows the positions (the chunk entry points), and NaN in the rotated channels where they
 * live in device memory (the step buffer, the pos arrays). */
int hipml_rope_set_table(const float *dev_table, float theta_base, int n_rot, int max_pos);
/* Opt in (allow != 0) to f64 pow/sincos on the device for positions outside the table: within one
 * f32 ulp of the host's values, not guaranteed identical to them.  Off by default. */
int hipml_rope_allow_device_angles(int allow);

/* M-RoPE over [n_heads][head_dim] at the four position ids in device memory
 * pos[0..3] (the step buffer's words 4..7).  x and y may alias.
 * Replaces AttnLayer::rope_launch -> mrope_f32,
 * crates/hipml-kernels/src/attn_gpu.rs:429-464. */
int hipml_mrope_f32(hipml_stream_t stream, const float *x, float *y, int n_heads, int head_dim,
                    int n_rot, int s0, int s1, int s2, int s3, const int32_t *pos,
                    float theta_base);
/* Same for `rows` rows of [n_heads][head_dim]; row r rotates at the text
 * position pos[r*2] (all four ids equal).  Replaces mrope_b,
 * crates/hipml-kernels/src/attn_gpu.rs:729-784. */
int hipml_mrope_rows_f32(hipml_stream_t stream, const float *x, float *y, int n_heads,
                         int head_dim, int n_rot, int s0, int s1, int s2, int s3,
                         const int32_t *pos, int rows, float theta_base);
/* RoPE of a prefill chunk in place: q [tokens][n_head][head_dim] and
 * k [tokens][n_kv][head_dim], token t at position pos0+t.  The RoPE half of
 * norm_rope_chunk_f32 (AttnLayer::chunk_front,
 * crates/hipml-kernels/src/attn_gpu/imp/attn_chunk.rs:167-199). */
int hipml_rope_chunk_f32(hipml_stream_t stream, float *q, float *k, int n_head, int n_kv,
                         int head_dim, int n_rot, float theta_base, int pos0, int tokens);

/* ---- attention front end ----------------------------------------------------- */

/* One token: split the joint projection qg [n_heads][2*head_dim] into q and gate
 * [n_heads][head_dim], RMS-normalise every q head and (in place) every k head
 * [n_kv][head_dim] with the shared weight rows q_norm / k_norm [head_dim], then
 * M-RoPE both with the four position ids at `pos` (device int32[4]).  Bit-identical
 * to the reference's kernel: squares folded by its 256-wide halving tree,
 * scale = 1/sqrtf(mean + eps), (x*scale)*w, f64 angles.  head_dim must be 256.
 * Replaces AttnLayer::front -> attn_front_f32 (= qg_split_f32 + head_rmsnorm_f32 x2
 * + mrope_f32 x2), crates/hipml-kernels/src/attn_gpu.rs:549-609,
 * crates/hipml-kernels/kernels/attn_front_f32.hip:34-135. */
int hipml_attn_front_f32(hipml_stream_t stream, const float *qg, float *q, float *gate, float *k,
                         const float *q_norm, const float *k_norm, int n_heads, int n_kv,
                         int head_dim, int n_rot, int s0, int s1, int s2, int s3,
                         const int32_t *pos, float theta_base, float eps);

/* The same over a chunk of `tokens` rows (qg [tokens][n_heads][2*head_dim], k
 * [tokens][n_kv][head_dim] in place); row t rotates at text position pos0 + t.
 * Argument order of the reference's launcher.  Replaces AttnLayer::chunk_front ->
 * qg_split_chunk_f32 + norm_rope_chunk_f32,
 * crates/hipml-kernels/src/attn_gpu/imp/attn_chunk.rs:129-205,
 * crates/hipml-kernels/kernels/attn_chunk_f32.hip:22-98. */
int hipml_attn_chunk_front_f32(hipml_stream_t stream, const float *qg, float *k, float *q,
                               float *gate, const float *q_norm, const float *k_norm, int n_heads,
                               int n_kv, int head_dim, int n_rot, float theta_base, float eps,
                               int pos0, int tokens);

/* hipml_attn_front_f32 and hipml_kv_encode (below) of the same token in one launch: the K row is
 * quantized from the registers that hold it after the rotation, the V row [n_kv][head_dim] by n_kv
 * more waves; q, gate, k and both caches end with the bits of the two calls.  `step` is the step
 * buffer (int32[8]): the row goes to position step[0], the M-RoPE position ids are step[4..7].
 * Replaces AttnLayer::front followed by Launcher::kv_encode_ptr_on
 * (crates/hipml-kernels/src/attn_gpu.rs:549-609, launch/device/graph_launch.rs:878-966; call site
 * crates/hipml-model/src/gpu.rs:576-592). */
int hipml_attn_front_encode_f32(hipml_stream_t stream, const int32_t *step, int dtype, const float *qg,
                                float *q, float *gate, float *k, const float *v, const float *q_norm,
                                const float *k_norm, void *k_cache, void *v_cache, int n_heads, int n_kv,
                                int head_dim, int n_rot, int s0, int s1, int s2, int s3, float theta_base,
                                float eps, int stride);

/* hipml_attn_chunk_front_f32 and hipml_kv_encode_bulk(start = pos0, src0 = 0, rows = tokens) in one
 * launch, same bits.  Replaces AttnLayer::chunk_front followed by Launcher::kv_encode_bulk
 * (crates/hipml-kernels/src/attn_gpu/imp/attn_chunk.rs:129-205,
 * launch/device/graph_launch.rs:980-1028; call site crates/hipml-model/src/gpu/attn_tile.rs:53-68). */
int hipml_attn_chunk_front_encode_f32(hipml_stream_t stream, int dtype, const float *qg, float *k,
                                      const float *v, float *q, float *gate, const float *q_norm,
                                      const float *k_norm, void *k_cache, void *v_cache, int n_heads,
                                      int n_kv, int head_dim, int n_rot, float theta_base, float eps,
                                      int pos0, int tokens, int stride);

/* The front end over the rows of a batch of sequences: row r rotates at text position pos[2 r]
 * (pos is the device int32 [rows][2] = (position, live length) the batched attention reads).  Same
 * arithmetic as hipml_attn_chunk_front_f32, whose row t sits at pos0 + t.  Replaces
 * AttnLayer::split_rope_rows -> qg_split_b + head_rmsnorm_b (q, k) + mrope_b (q, k),
 * crates/hipml-kernels/src/attn_gpu.rs:649-784; call site crates/hipml-model/src/gpu/batch/forward.rs:79-88. */
int hipml_attn_front_rows_f32(hipml_stream_t stream, const float *qg, float *k, float *q, float *gate,
                              const float *q_norm, const float *k_norm, int n_heads, int n_kv,
                              int head_dim, int n_rot, float theta_base, float eps, const int32_t *pos,
                              int rows);

/* hipml_attn_front_rows_f32 and hipml_kv_encode_rows (below) of the same step in one launch, same
 * bits: row r's K and V go to position pos[2 r] of sequence r's cache, which starts r * slot_bytes
 * into k_cache / v_cache.  Replaces split_rope_rows followed by Launcher::kv_encode_batch
 * (crates/hipml-model/src/gpu/batch/forward.rs:79-106). */
int hipml_attn_front_rows_encode_f32(hipml_stream_t stream, int dtype, const float *qg, float *k,
                                     const float *v, float *q, float *gate, const float *q_norm,
                                     const float *k_norm, void *k_cache, void *v_cache, int n_heads,
                                     int n_kv, int head_dim, int n_rot, float theta_base, float eps,
                                     int stride, const int32_t *pos, size_t slot_bytes, int slots);

/* ---- q8_0 / q4_0 KV append ------------------------------------------------------- */

/* One token: quantize k_in/v_in [n_kv][head_dim] into row step[0] of the cache.
 * Replaces Launcher::kv_encode_ptr_on -> kv_encode_q8,
 * crates/hipml-kernels/src/launch/device/graph_launch.rs:932-973. */
int hipml_kv_encode(hipml_stream_t stream, const int32_t *step, int dtype, const float *k_in,
                    const float *v_in, void *k_cache, void *v_cache, int n_kv, int head_dim,
                    int stride);
/* `rows` tokens from position-major f32 [.][n_kv*head_dim]; source row src0+r
 * goes to cache position start+r.  Replaces Launcher::kv_encode_bulk ->
 * kv_encode_bulk_q8, graph_launch.rs:980-1028. */
int hipml_kv_encode_bulk(hipml_stream_t stream, int dtype, const float *k_f32, const float *v_f32,
                         void *k_cache, void *v_cache, int n_kv, int head_dim, int stride,
                         int start, int src0, int rows);
/* RoPE of a chunk and the append of its K/V rows in one launch: hipml_rope_chunk_f32(q, k, ...)
 * followed by hipml_kv_encode_bulk(dtype, k, v, ..., start = pos0, src0 = 0, rows = tokens), with the
 * same bits in q, k and both caches.  v is f32 [tokens][n_kv][head_dim].  head_dim 256, n_rot 64.
 * q may be NULL: then only the K rows are rotated (for hipml_attn_chunk_rope_q8, which rotates the
 * query rows itself).
 * Replaces the RoPE half of AttnLayer::chunk_front + Launcher::kv_encode_bulk as issued per chunk,
 * crates/hipml-model/src/gpu/attn_tile.rs:53-68. */
int hipml_rope_encode_chunk_f32(hipml_stream_t stream, float *q, float *k, const float *v, void *k_cache,
                                void *v_cache, int n_head, int n_kv, int head_dim, int n_rot,
                                float theta_base, int pos0, int tokens, int dtype, int stride);

/* One row per slot: row s of k_f32/v_f32 goes to cache (base + s*slot_bytes) at
 * position pos[s*2].  Replaces Launcher::kv_encode_rows_ptr -> kv_encode_q8_b,
 * crates/hipml-kernels/src/launch/device/batch_launch.rs:59-105. */
int hipml_kv_encode_rows(hipml_stream_t stream, int dtype, const float *k_f32, const float *v_f32,
                         void *k_cache, void *v_cache, int n_kv, int head_dim, int stride,
                         const int32_t *pos, size_t slot_bytes, int slots);

/* ---- decode attention over a q8_0 / q4_0 cache -----------------------------------
 * head_dim is 256 (the MFMA kernels) or 64: the reference's launchers take any multiple of the block
 * size and its parity table runs 64 (crates/hipml-core/src/parity_kv.rs:166-213); that width is
 * served by plain fp32 kernels behind the same arguments, untuned (hipml_attn_decode_kv_noalloc: 256
 * only).  Other widths are HIPML_ATTN_E_SHAPE. */

/* One query row, live length step[1].  Split pass + merge.
 * part_acc: f32 [n_heads][splits][head_dim]; part_ml: f32 [n_heads][splits][2].
 * Replaces launch_kv::launch_ptrs -> attn_decode_kv_w2 + attn_decode_kv_reduce,
 * crates/hipml-kernels/src/launch_kv.rs:110-280. */
int hipml_attn_decode_kv(hipml_stream_t stream, const int32_t *step, int dtype, const float *q,
                         const void *k, const void *v, float *part_acc, float *part_ml,
                         float *out, int n_heads, int n_kv, int head_dim, int stride, float scale,
                         int splits, size_t k_off, size_t v_off);
/* `cols` (<= 4) consecutive query rows of ONE sequence sharing the cache
 * (MTP verify): column c reads q + c*q_slot, sees keys [0, pos[c*2+1]), writes
 * out + c*q_slot, and owns scratch slices part_acc + c*acc_slot and
 * part_ml + c*ml_slot (all in f32 elements).  The cache is streamed once for
 * all columns.  Replaces launch_kv::launch_cols_ptrs -> attn_decode_kv_w2_b +
 * attn_decode_kv_reduce_b, crates/hipml-kernels/src/launch_kv.rs:292-412. */
int hipml_attn_decode_kv_cols(hipml_stream_t stream, int dtype, const int32_t *pos,
                              const float *q, const void *k, const void *v, float *part_acc,
                              float *part_ml, float *out, int n_heads, int n_kv, int head_dim,
                              int stride, float scale, int splits, int cols, size_t acc_slot,
                              size_t ml_slot, size_t q_slot);
/* `slots` independent rows: row s reads cache base + s*kv_slot_bytes, q +
 * s*q_slot, keys [0, pos[s*2+1]).  kv_slot_bytes == 0 means the rows share one
 * cache (a verify group).  Replaces Launcher::attn_decode_rows_ptr ->
 * attn_decode_kv_q8_b + attn_decode_kv_reduce_b,
 * crates/hipml-kernels/src/launch/device/batch_launch.rs:215-316. */
int hipml_attn_decode_rows(hipml_stream_t stream, int dtype, const int32_t *pos, const float *q,
                           const void *k_cache, const void *v_cache, float *part_acc,
                           float *part_ml, float *out, int n_heads, int n_kv, int head_dim,
                           int stride, float scale, int splits, size_t kv_slot_bytes,
                           size_t acc_slot, size_t ml_slot, size_t q_slot, int slots);
/* Batched decode step.  `live_seq` > 0 with slots == 1 states a plain decode
 * step at a known length (the reference reroutes that case to its warp kernel;
 * here both cases run the same kernel and the value is only validated).
 * Replaces Launcher::attn_decode_batch, batch_launch.rs:109-213. */
int hipml_attn_decode_batch(hipml_stream_t stream, int dtype, const int32_t *pos, const float *q,
                            const void *k_cache, const void *v_cache, float *part_acc,
                            float *part_ml, float *out, int n_heads, int n_kv, int head_dim,
                            int stride, float scale, int splits, size_t kv_slot_bytes,
                            size_t acc_slot, size_t ml_slot, size_t q_slot, int slots,
                            int live_seq);
/* Batched decode where slot s carries cols_per_slot[s] (1..4) consecutive query
 * rows that share slot s's cache (plain slots and MTP-verify slots mixed in ONE
 * launch).  Rows are numbered slot-major: row r has (pos,seq) = pos[r*2..],
 * q + r*q_slot, scratch r*acc_slot / r*ml_slot; slot s's cache is base +
 * s*kv_slot_bytes.  cols_per_slot is a HOST array read during the call: the rows per slot
 * become part of the launch (its grid and item tables), so a graph captured around this
 * call replays that layout; positions and live lengths stay device data and may change
 * between replays.
 * The reference has no single-launch form of this: it issues one launch pair
 * per verify slot (crates/hipml-model/src/gpu/batch/verify.rs:321-366). */
int hipml_attn_decode_batch_cols(hipml_stream_t stream, int dtype, const int32_t *pos,
                                 const float *q, const void *k_cache, const void *v_cache,
                                 float *part_acc, float *part_ml, float *out, int n_heads,
                                 int n_kv, int head_dim, int stride, float scale, int splits,
                                 size_t kv_slot_bytes, size_t acc_slot, size_t ml_slot,
                                 size_t q_slot, int slots, const int32_t *cols_per_slot_host);

/* Decode with the sigmoid output gate applied where the splits are merged:
 * out = attention * sigmoid(gate), `gate` laid out like `out` (f32 [n_heads][head_dim] per row,
 * rows q_slot apart).  The result has the bits of the ungated call followed by hipml_q_gate_f32
 * on the same rows; it saves that launch.  hipml_attn_decode_kv_gate is
 * hipml_attn_decode_kv (one row, position from the step buffer) and
 * hipml_attn_decode_batch_cols_gate is hipml_attn_decode_batch_cols, each with `gate` after `out`.
 * Replaces launch_kv::launch_ptrs / attn_decode_batch followed by AttnLayer::q_gate_only or the
 * gate half of output_rows, crates/hipml-kernels/src/attn_gpu.rs:822-840,967-990. */
int hipml_attn_decode_kv_gate(hipml_stream_t stream, const int32_t *step, int dtype, const float *q,
                              const void *k, const void *v, float *part_acc, float *part_ml,
                              float *out, const float *gate, int n_heads, int n_kv, int head_dim,
                              int stride, float scale, int splits, size_t k_off, size_t v_off);
int hipml_attn_decode_batch_cols_gate(hipml_stream_t stream, int dtype, const int32_t *pos,
                                      const float *q, const void *k_cache, const void *v_cache,
                                      float *part_acc, float *part_ml, float *out,
                                      const float *gate, int n_heads, int n_kv, int head_dim,
                                      int stride, float scale, int splits, size_t kv_slot_bytes,
                                      size_t acc_slot, size_t ml_slot, size_t q_slot, int slots,
                                      const int32_t *cols_per_slot_host);

/* hipml_attn_decode_kv for callers that cannot allocate or bring scratch: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference (whose callers own part_acc / part_ml, crates/hipml-model/src/gpu/deep_kv.rs:80-81).
 * The split partials live in an array built into the library (one copy of 4,227,072 bytes per GPU
 * the library has been initialised on, held until the process ends); the call allocates nothing and
 * frees nothing.  Limit: n_heads * splits <= 4096, else HIPML_ATTN_E_RANGE.  Same kernels, same
 * bits in `out` as hipml_attn_decode_kv.  All calls on one GPU share the array: calls that overlap
 * on one GPU (two streams, or a captured graph replayed while another call runs) race; calls on one
 * stream are ordered and safe.  Nothing in the array has to be cleared between calls. */
int hipml_attn_decode_kv_noalloc(hipml_stream_t stream, const int32_t *step, int dtype, const float *q,
                                 const void *k, const void *v, float *out, int n_heads, int n_kv,
                                 int head_dim, int stride, float scale, int splits, size_t k_off,
                                 size_t v_off);

/* How a single sequence over a q8_0 cache (hipml_attn_decode_kv, _gate, _noalloc, _cols) merges its key
 * splits.  0 (the default): a second launch, as in the reference (attn_decode_kv_reduce,
 * crates/hipml-kernels/kernels/attn_decode_kv.hip:491-532).  1: the workgroups of the one launch merge
 * them: each takes a ticket when its partial is in memory, the last of eight neighbouring splits folds
 * those, the last of those groups folds the groups and writes `out`; nobody waits, nothing is allocated
 * (the counters are library memory, one set per stream for the first 32 streams of a device and a ring
 * of 96 for launches under capture; launches that share a set must not overlap).  Same tolerance class,
 * not the same bits as mode 0; a verify column still has the bits of its row's plain decode in the same
 * mode.  Measured on MI355X it is the slower form at every depth (depth 32,768: 23.3 against 20.0 us
 * per layer; 8,192: 15.7 against 11.4; 673: 10.1 against 9.6): one level of such a merge is three
 * dependent device-scope round trips of ~1.2 us, as much as the launch it saves.  It has no counterpart
 * in the reference and is kept so that this figure can be measured again.  on < 0 only reads the mode;
 * returns the mode before the call.  Environment: HIPML_DECODE_ONE_LAUNCH=1 sets the initial mode. */
int hipml_attn_decode_one_launch(int on);

/* ---- causal chunk prefill over a q8_0 / q4_0 cache -------------------------------- */

/* tokens query rows at positions pos0..pos0+tokens-1 attend keys [0, pos0+t]
 * of a cache that already holds the chunk's own rows.  `dtype` follows the
 * reference's chunk launcher: 1 = q8_0, 2 = q4_0.  splits == 1 runs the single-pass kernel
 * and splits == 0 the kernel that cuts the keys into four slices inside each workgroup (one
 * workgroup per 32 tokens x 2 heads; made for chunks near position 0, correct at any depth);
 * both ignore the scratch.  Otherwise part_acc is f32
 * [splits][ceil32(tokens)][n_head][head_dim] and part_ml [..][2]; how that memory is used is the
 * library's business (with a count from hipml_attn_chunk_splits for a long chunk behind a prefix,
 * fewer slices run and the rest of part_acc holds the cache rows as f16 tiles for the length of the
 * call), and nothing beyond those sizes is touched.
 * Replaces AttnLayer::chunk_attention_q8_split -> attn_chunk_wmma_f16 /
 * attn_chunk_full_f16 + attn_chunk_combine_f32,
 * crates/hipml-kernels/src/attn_gpu/imp/attn_chunk_kv.rs:72-107,129-305. */
int hipml_attn_chunk_q8_split(hipml_stream_t stream, const float *q, const void *kc,
                              const void *vc, float *out, int n_head, int n_kv, int head_dim,
                              int pos0, int tokens, int dtype, int stride, float *part_acc,
                              float *part_ml, int splits);

/* The same attention with the sigmoid output gate applied where the result is
 * written (in the key-slice merge, or in the attention kernel for rows that are
 * not sliced): out = attention * sigmoid(gate), gate f32 [tokens][n_head][head_dim].
 * Bit-identical to hipml_attn_chunk_q8_split followed by hipml_q_gate_f32 on its
 * output; it saves that kernel's pass over the rows.  Replaces the pair
 * AttnLayer::chunk_attention_q8_split (attn_chunk_kv.rs:72-107) + q_gate_only
 * (crates/hipml-kernels/src/attn_gpu.rs:822-834) of the reference's chunk path. */
int hipml_attn_chunk_q8_split_gate(hipml_stream_t stream, const float *q, const void *kc,
                                   const void *vc, const float *gate, float *out, int n_head,
                                   int n_kv, int head_dim, int pos0, int tokens, int dtype,
                                   int stride, float *part_acc, float *part_ml, int splits);

/* The same with the finished rows delivered as f16 (round to nearest even) in out16
 * [tokens][n_head][head_dim], 16-byte aligned: the operand form of the output projection, so
 * hipml_attn_output_chunk_q8_0(attn_out = NULL, gate = NULL, x16 = out16) can follow without its
 * conversion pass.  out16 holds exactly f16(what hipml_attn_chunk_q8_split_gate writes to out);
 * `out` (same size as there) is working memory here and holds nothing defined afterwards.
 * Replaces chunk_attention_q8_split + apply_output_chunk's gate
 * (attn_chunk_kv.rs:72-107, crates/hipml-kernels/src/attn_gpu/imp/attn_chunk.rs:343-364). */
int hipml_attn_chunk_q8_split_gate_f16(hipml_stream_t stream, const float *q, const void *kc,
                                       const void *vc, const float *gate, float *out, void *out16,
                                       int n_head, int n_kv, int head_dim, int pos0, int tokens, int dtype,
                                       int stride, float *part_acc, float *part_ml, int splits);

/* hipml_rope_chunk_f32 of the query rows and the chunk attention in one call: q holds the
 * UNROTATED query rows.  With splits == 0 (and n_rot 64, positions inside the registered table) the
 * attention kernel rotates each row between its load and its use, with the expressions of the RoPE
 * kernels, and q is left as it was: the pass that rotates the query rows in memory (33 MB of traffic
 * for 672 tokens) goes away; pair it with hipml_rope_encode_chunk_f32(q = NULL), which rotates and
 * appends the K rows only.  With any other `splits` the rows are first rotated in place
 * (hipml_rope_chunk_f32 on q alone) and the call continues as hipml_attn_chunk_q8_split_gate /
 * _gate_f16; q then holds the rotated rows.  Either way the results are the bits of the separate
 * calls.  gate and out16 may be NULL (no gate / f32 rows in `out`); with out16 the rows are
 * delivered as f16 there and `out` is working memory.  Replaces the query half of the RoPE in
 * norm_rope_chunk_f32 (AttnLayer::chunk_front, crates/hipml-kernels/src/attn_gpu/imp/attn_chunk.rs:167-199)
 * followed by chunk_attention_q8_split (attn_chunk_kv.rs:72-107). */
int hipml_attn_chunk_rope_q8(hipml_stream_t stream, float *q, const void *kc, const void *vc,
                             const float *gate, float *out, void *out16, int n_head, int n_kv,
                             int head_dim, int n_rot, float theta_base, int pos0, int tokens, int dtype,
                             int stride, float *part_acc, float *part_ml, int splits);

/* ---- chunk prefill over an f16 copy of the cache -------------------------------------------------
 * The reference's chunk kernel dequantizes the cache rows it attends over inside every workgroup
 * (crates/hipml-kernels/kernels/attn_chunk_wmma.hip:187-399), and so do the entry points above: at a
 * long prefix that is 40 % of the kernel's vector instructions, done once per 256 (token, head)
 * pairs.  These three have no counterpart in the reference.  They keep a second form of a layer's
 * cache, f16(d * q) of every K and V value (exactly the operands the kernels above compute), laid
 * out in 64-key tiles the way the attention kernel wants them in LDS, K rows as they are and V
 * transposed; the attention kernel then copies whole tiles and spends its vector instructions on
 * the softmax alone.  The copy costs hipml_kv_f16_bytes(stride, n_kv) = n_kv * ceil(stride / 64) *
 * 70,656 bytes per layer cache (450 MB for 102,048 rows) and is kept up to date by the caller: after
 * appending rows [start, start + rows) to the cache, call hipml_kv_f16_rows for the same rows.  It
 * rewrites every 64-key tile that holds one of them from the tile's first row on, so a partly
 * filled tile is completed by the next call; rows of a tile at or past start + rows hold copies
 * of row start + rows - 1.  One copy can also be shared by all layers and rebuilt from row 0
 * before each layer's attention (start = 0, rows = pos0 + tokens: one pass over the cache).
 * dtype is the KvDtype id of the cache, as for the append entry points (0 = q8_0, 1 = q4_0).
 * kv_f16 is 16-byte aligned device memory of at least hipml_kv_f16_bytes(stride, n_kv). */
size_t hipml_kv_f16_bytes(int stride, int n_kv);
int hipml_kv_f16_rows(hipml_stream_t stream, int dtype, const void *k_cache, const void *v_cache,
                      void *kv_f16, int n_kv, int head_dim, int stride, int start, int rows);

/* hipml_attn_chunk_q8_split (splits >= 2, with scratch) or hipml_attn_chunk_q8 (splits <= 1) over the
 * copy: rows [0, pos0 + tokens) of kv_f16 must be current.  gate (may be NULL) and out16 (may be NULL)
 * as in hipml_attn_chunk_q8_split_gate / _gate_f16.  The operands are the same values, so results
 * differ from those entry points only through the key slices, which here end at multiples of 64
 * keys.  Same scratch sizes; slice counts from hipml_attn_chunk_slices (splits == 0 is taken as 1:
 * there is no in-workgroup variant over the copy). */
int hipml_attn_chunk_kv_f16(hipml_stream_t stream, const float *q, const void *kv_f16,
                            const float *gate, float *out, void *out16, int n_head, int n_kv,
                            int head_dim, int pos0, int tokens, int stride, float *part_acc,
                            float *part_ml, int splits);

/* The same copy kept by the library, behind the reference's own entry points.  hipml_kv_f16_attach registers
 * kv_f16 (hipml_kv_f16_bytes(stride, n_kv) bytes, 16-byte aligned) as the f16 shadow of the cache
 * (k_cache, v_cache) and converts its rows [0, rows) on `stream`.  From then on, without any change to the
 * calls the reference's engine makes per chunk (crates/hipml-model/src/gpu/attn_tile.rs:53-82):
 *   - the entry points that write rows of that cache at positions the host knows (hipml_kv_encode_bulk,
 *     hipml_rope_encode_chunk_f32, hipml_attn_chunk_front_encode_f32, hipml_kv_rows_copy as destination)
 *     convert those rows right behind their own launch;
 *   - the ones whose positions live in device memory (hipml_kv_encode, hipml_attn_front_encode_f32,
 *     hipml_kv_encode_rows, hipml_attn_front_rows_encode_f32) mark the shadow stale, and the next chunk
 *     attention over the cache converts every live row once (0.13 ms per 100,000 rows);
 *   - hipml_attn_chunk_q8_split, _gate and _gate_f16 over (k_cache, v_cache) with the registered stride,
 *     n_kv and format and splits >= 2 read the tiles: min(splits, hipml_attn_chunk_slices) slices, no
 *     tiles made per call in the scratch (2,048 tokens at depth 100,000: 4.06 against 4.19 ms).
 * The bookkeeping is host state that changes when a call is issued or captured, not when a captured
 * graph is replayed.  Rows written into the cache by any other means (a device copy, another library)
 * must be followed by hipml_kv_f16_rows for those rows.  hipml_kv_f16_detach must be called before
 * either buffer is freed; it is HIPML_ATTN_E_STATE for a cache that has no shadow.  At most 1,024 caches
 * per process.  No counterpart in the reference: its DeepKv::new (crates/hipml-model/src/gpu/deep_kv.rs:41-83)
 * is where an engine would allocate the copy and attach it. */
int hipml_kv_f16_attach(hipml_stream_t stream, int dtype, const void *k_cache, const void *v_cache,
                        void *kv_f16, int n_kv, int head_dim, int stride, int rows);
int hipml_kv_f16_detach(const void *k_cache);

/* ---- output gate ------------------------------------------------------------ */

/* y[i] = x[i] * sigmoid(gate[i]); y may alias x.  Replaces
 * AttnLayer::q_gate_only / apply_output_chunk -> q_gate_f32,
 * crates/hipml-kernels/src/attn_gpu.rs:822-840 and
 * crates/hipml-kernels/src/attn_gpu/imp/attn_chunk.rs:343-364. */
int hipml_q_gate_f32(hipml_stream_t stream, const float *x, const float *gate, float *y,
                     size_t n);

/* Prefix snapshot / restore: rows [0, rows) of every KV head of K and V, from a cache with
 * src_stride rows per head to one with dst_stride rows per head (same format; dtype 0 = q8_0,
 * 1 = q4_0).  dst_stride = rows packs a prefix as [head][rows][row bytes]; swapping the roles
 * restores it.  One launch, asynchronous, legal under capture.
 * Replaces the per-head copy_range_on loop of GpuEngine::prefix_capture / prefix_restore over a
 * DeepKv, crates/hipml-model/src/gpu/prefix.rs:214-239. */
int hipml_kv_rows_copy(hipml_stream_t stream, int dtype, const void *k_src, const void *v_src, void *k_dst,
                       void *v_dst, int n_kv, int head_dim, int src_stride, int dst_stride, int rows);

/* ---- projections over Q8_0 weight matrices (the steps either side of the attention core) ---- */

/* y[r][row] = sum_k W[row][k] * x[r][k] for r < rows: W is m rows of k/32 Q8_0 blocks (34 bytes:
 * f16 scale, 32 int8) at a 4-byte aligned address, x is f32 [rows][k] (16-byte aligned), y is f32
 * [rows][m]; k a multiple of 64 up to 32768, 1 <= rows <= 128.
 * fp32 accumulation of exact integer block products (the activations enter as hi + lo f16 halves), so
 * every row has the precision class of the reference's f32 GEMV kernels.  Up to 8 rows W streams from
 * memory once and a row's result has the same bits whatever `rows` is and whichever rows travel with it:
 * the rows of a verify group match their plain decodes, as the reference's batched GEMVs do
 * (crates/hipml-kernels/src/attn_gpu.rs:930-932).  From 10 to 128 rows W streams once per pass of up to 64 rows
 * (two passes beyond 64) and a row's bits are the same for every such `rows`; 9 rows take a kernel of their own.
 * The three classes differ from each other in the last bits.
 * (W at a 16-byte aligned address and k a multiple of 256 take the fastest road.)
 * Replaces AttnLayer::gemv / gemv_rows / gemv_batched over a Q8_0 ResidentMat (the output
 * projection of apply_output / output_rows, and W_q, W_k, W_v in prepare_rows),
 * crates/hipml-kernels/src/attn_gpu.rs:843-846,967-1023,1066-1117 -> gemv_q8_0 / gemv_q8_0_b,
 * crates/hipml-kernels/kernels/gemv_q8_0.hip:20-66. */
int hipml_gemv_q8_0_rows(hipml_stream_t stream, const void *w, const float *x, float *y, int m,
                         int k, int rows);

/* The same product for a prefill chunk (any number of tokens): y[t][row] = W[row][:] . x[t][:] on
 * MFMA with f16 operands -- x rounded to f16, W dequantized to f16(d*q) -- and fp32 accumulation:
 * the precision class of the reference's f16-operand prefill kernels (its f32 tile kernel for Q8_0
 * is bounded by 1e-4 on small cases; this one by 2e-3 abs / 3e-2 rel, the reference's LARGE_TOL, at
 * the model's shape).  Same layouts and argument rules as hipml_gemv_q8_0_rows.
 * Replaces AttnLayer::apply_output_chunk -> prefill_resident(prefill_q8_0) after the gate, and the
 * chunk's Q/K/V projections, crates/hipml-kernels/src/attn_gpu/imp/attn_chunk.rs:343-397,
 * crates/hipml-kernels/kernels/prefill_q8_0.hip:44-60. */
int hipml_gemm_q8_0_f16(hipml_stream_t stream, const void *w, const float *x, float *y, int m, int k,
                        int tokens);

/* The output side of a chunk in one call: y = W_o (attn_out * sigmoid(gate)), gate may be NULL (the
 * rows are already gated, e.g. by hipml_attn_chunk_q8_split_gate).  x16 is caller scratch of
 * tokens*k f16 (2 bytes each, 16-byte aligned; the attention's split scratch is free by then): a
 * first kernel gates and rounds the rows to f16 once, the GEMM then reads half the bytes per
 * workgroup.  Same bits as hipml_q_gate_f32 followed by hipml_gemm_q8_0_f16, faster.
 * attn_out == NULL (then gate must be NULL too): x16 already holds the rows as f16, as
 * hipml_attn_chunk_q8_split_gate_f16 writes them, and only the GEMM runs.
 * Replaces AttnLayer::apply_output_chunk (q_gate_f32 + the tiled GEMM),
 * crates/hipml-kernels/src/attn_gpu/imp/attn_chunk.rs:343-397. */
int hipml_attn_output_chunk_q8_0(hipml_stream_t stream, const void *wo, const float *attn_out,
                                 const float *gate, float *y, int m, int k, int tokens, void *x16);

/* ---- measurement only: yardsticks for the benchmark ----------------------------------------------
 * Not part of the attention path and without a counterpart in the reference's launchers; they stand where the
 * reference's bandwidth probes do (crates/hipml-kernels/kernels/bw_probe.hip, stream_read.hip, printed beside
 * every decode figure by crates/hipml-kernels/src/kvbench.rs:209-249).  Both launch asynchronously on
 * `stream`, allocate nothing and write at most the few bytes named below. */

/* One launch of 256 workgroups that reads bytes_each bytes (a positive multiple of 8,704 = 32 cache rows)
 * of each of `a` and `b` once, dealt to workgroups and waves as the decode kernel deals the K and V rows of
 * a cache, and does nothing with them.  mode 0: global memory straight into LDS (global_load_lds_dwordx4,
 * non-temporal), the decode kernel's road; mode 1: non-temporal 128-bit loads into registers.  `sink`:
 * 4 bytes of device memory (never written in practice; it keeps the loads alive). */
int hipml_bench_stream_read(hipml_stream_t stream, const void *a, const void *b, size_t bytes_each, int mode,
                            void *sink);
/* `workgroups` workgroups of four waves, one per SIMD, each wave issuing iters x 8 independent
 * v_mfma_f32_32x32x16_f16: workgroups x 4 x iters x 8 x 32,768 FLOP per launch.  `sink`: 4 bytes of device
 * memory (as above).  `clocks`: NULL or 16 bytes of device memory that receive, from one wave, the core
 * clock cycles and the ticks of the constant 100 MHz counter its loop took (the clock the chip ran at
 * under this load is their ratio x 100 MHz). */
int hipml_bench_mfma_f16(hipml_stream_t stream, int workgroups, int iters, void *sink, void *clocks);

#ifdef __cplusplus
}
#endif
#endif /* HIPML_ATTN_H */
