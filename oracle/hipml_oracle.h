/*
 * CPU oracle for the hipml full-attention hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's CPU definitions (the files named
 * beside each prototype are paths inside the reference repository).  It exists
 * so the HIP kernels can be checked on identical seeded inputs; nothing the
 * library ships may call it.  Only tests, the smoke check and the CPU-baseline
 * leg of the benchmark load it.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math (no value-changing options),
 * so the summation order written here is the summation order executed.
 *
 * Parity status: every function below is pinned by the reference's own
 * known-answer tests and by closed forms (see tests/test_oracle_*.py), except
 * the bit patterns of orc_rng_normal(), which depend on the platform's
 * logf/cosf and are not stored anywhere in the reference ("parity unpinned";
 * harmless: both sides of every comparison consume the same generated array).
 */
#ifndef HIPML_ORACLE_H
#define HIPML_ORACLE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_Q8 = 0, ORC_Q4 = 1, ORC_BLOCK = 32 };

/* crates/hipml-core/src/kv.rs:47-91 */
size_t orc_block_bytes(int dtype);
size_t orc_row_bytes(int dtype, size_t head_dim);
size_t orc_token_bytes(int dtype, size_t n_kv, size_t head_dim, size_t n_layers);
/* kv.rs:94-165 */
float orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_f16(float v);
/* kv.rs:176-235 */
void orc_quantize_block(int dtype, const float *xs, uint8_t *out);
void orc_quantize(int dtype, const float *values, size_t n_values, uint8_t *out);
/* kv.rs:238-290 */
void orc_block_f32(int dtype, const uint8_t *src, float *out32);
void orc_dequantize(int dtype, const uint8_t *bytes, size_t n_bytes, float *out);
/* kv.rs:306-329 */
void orc_synthetic_blocks(int dtype, size_t n_blocks, uint64_t seed, uint8_t *out);

/* crates/hipml-core/src/rng.rs:9-50 */
typedef struct { uint64_t state; } orc_rng;
void orc_rng_new(orc_rng *r, uint64_t seed);
uint64_t orc_rng_next_u64(orc_rng *r);
float orc_rng_uniform(orc_rng *r);
float orc_rng_normal(orc_rng *r);
/* Tensor::from_fn(|_| rng.normal_scaled(std)) in row-major order,
 * crates/hipml-core/src/tensor.rs:43-49 */
void orc_rng_fill_normal(orc_rng *r, float *out, size_t n, float std);
void orc_rng_fill_uniform(orc_rng *r, float *out, size_t n);

/* crates/hipml-core/src/ops.rs:62-64 */
void orc_sigmoid_f32(const float *x, float *out, size_t n);
/* ops.rs:195-224 */
void orc_rope_neox_f32(const float *x, float *y, size_t n_heads, size_t head_dim,
                       size_t pos, float theta_base);
/* ops.rs:260-309 */
void orc_rope_multi_f32(const float *x, float *y, size_t n_heads, size_t head_dim,
                        size_t n_rot, const size_t sections[4], const size_t pos[4],
                        float theta_base);
/* ops.rs:354-360 */
void orc_q_gate_f32(const float *q, const float *gate, float *y, size_t n);

/* attention front end (ops.rs:178-187, 315-349); `_tree` sums the squares in the order of the
 * reference's GPU kernels (one square per thread, shared-memory halving tree) */
void orc_rmsnorm_f32(const float *x, const float *w, float *y, size_t n, float eps);
void orc_head_rmsnorm_f32(const float *x, const float *w, float *y, size_t n_heads, size_t head_dim,
                          float eps);
void orc_rmsnorm_tree_f32(const float *x, const float *w, float *y, size_t n, float eps);
void orc_qg_split_f32(const float *qg, float *q, float *gate, size_t n_heads, size_t head_dim);
/* ops.rs:366-386 (in place on the two caches) */
void orc_kv_append_f32(float *k_cache, float *v_cache, const float *k, const float *v,
                       size_t off, size_t width);
/* crates/hipml-core/src/attention.rs:56-102 */
void orc_attn_causal_f32(const float *q, const float *k_cache, const float *v_cache,
                         size_t n_heads, size_t n_kv, size_t head_dim, size_t seq,
                         float scale, float *out);
/* ops.rs:535-588 */
void orc_attn_decode_f32(const float *q, const float *k, const float *v, size_t n_heads,
                         size_t n_kv, size_t head_dim, size_t seq, float scale, float *out);
/* ops.rs:449-518.  `stride` is the cache's rows per KV head; the reference
 * passes a cache of exactly `seq` rows (stride == seq). */
void orc_attn_decode_kv(const float *q, const uint8_t *k, const uint8_t *v, size_t n_heads,
                        size_t n_kv, size_t head_dim, size_t seq, size_t stride, float scale,
                        int dtype, float *out);
/* attention.rs:140-161, the part after the projections and head norms:
 * rope(q,k) at pos -> append -> attn_causal_f32(seq = pos+1) -> out *= sigmoid(gate). */
void orc_attn_core_token_f32(float *q, float *k, const float *v, const float *gate,
                             float *k_cache, float *v_cache, size_t n_ctx, size_t n_heads,
                             size_t n_kv, size_t head_dim, size_t n_rot,
                             const size_t sections[4], size_t pos, float theta_base,
                             float *out);
/* crates/hipml-cli/src/attn_chunk_parity.rs:127-210: the expected side of the
 * chunk-prefill case.  Row t = attn_causal_f32 over the DEQUANTIZED cache with
 * seq = pos0 + t + 1.  `rows` selects which chunk rows to compute (NULL = all);
 * out is [n_rows][n_heads][head_dim].  n_threads > 1 spreads rows over OpenMP
 * threads; each row is still the scalar single-thread arithmetic. */
void orc_attn_chunk_kv(const float *q, const uint8_t *k, const uint8_t *v, size_t n_heads,
                       size_t n_kv, size_t head_dim, size_t pos0, size_t tokens, size_t stride,
                       float scale, int dtype, const int32_t *rows, size_t n_rows,
                       int n_threads, float *out);
/* ---- Q8_0 weight matrices (the projections either side of the attention core) ------------
 * crates/hipml-core/src/quant.rs:433-443 (dequant_q8_0), :653-675 (gemv_q8_0),
 * crates/hipml-core/src/ops.rs:102-104,136-176 (gemm_q8_0), quant.rs:785-796,846-854
 * (random_q8_0_bytes: eight bytes per next_u64 little-endian, then the scale bytes overwritten
 * with f16 0x1400 = 2^-10). */
void orc_dequant_q8_0(const uint8_t *block, float *out);
/* y[m] = sum over blocks in order, within a block l = 0..31: acc += (d * q_l) * x_l. */
void orc_gemv_q8_0(const uint8_t *w, const float *x, size_t m, size_t k, float *y);
/* y[t][m]: the row is dequantized once, then acc += row[j] * x[t][j] for j ascending. */
void orc_gemm_q8_0(const uint8_t *w, const float *x, size_t tokens, size_t m, size_t k,
                   int n_threads, float *y);
void orc_random_q8_0_bytes(orc_rng *r, size_t nblocks, uint8_t *out);

/* crates/hipml-core/src/parity.rs:44-80.  Returns 1 when within tolerance
 * (max_abs <= abs_tol OR max_rel <= rel_tol). */
int orc_compare(const float *expected, const float *actual, size_t n, float abs_tol,
                float rel_tol, float *max_abs, float *max_rel);

#ifdef __cplusplus
}
#endif
#endif
