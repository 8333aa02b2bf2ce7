// Shared host-side helpers of libhipml_attn.so: status codes, the thread-local
// error text, argument checks.  Device code lives in the .hip files.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/hipml_attn.h"

namespace hipml {

constexpr int kBlock = 32;        // values per quantization block
constexpr int kQ8BlockBytes = 34; // f16 scale + 32 int8
constexpr int kQ4BlockBytes = 18; // f16 scale + 16 bytes of nibble pairs (j, j + 16)
constexpr int kHeadDim = 256;     // the width the MFMA kernels are built for
constexpr int kRowBytes = kHeadDim / kBlock * kQ8BlockBytes; // 272
constexpr int kRowBytesQ4 = kHeadDim / kBlock * kQ4BlockBytes; // 144
constexpr int kMaxCols = 4;       // query rows of one sequence per launch (MTP verify)
constexpr int kMaxSlots = 128;    // slots per batched launch
constexpr int kMaxGroup = 8;      // query heads per KV head

// Record `msg` for hipml_attn_last_error() and return `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// Translate the status of this thread's most recent HIPML_LAUNCH: the return code of that launch call itself,
// so an error the caller's own earlier HIP calls left pending is neither consumed nor mistaken for ours.
int launched(const char *what);
void set_launch_status(hipError_t e);
void clear_error();

#ifdef __HIPCC__
} // namespace hipml
#include <tuple>
#include <utility>
namespace hipml {
template <typename Tuple, size_t... I>
inline void launch_pointers(Tuple &vals, void **ptrs, std::index_sequence<I...>)
{
    ((ptrs[I] = static_cast<void *>(&std::get<I>(vals))), ...);
}
// kernel<<<grid, block, lds, st>>>(args...) with the status kept for launched().
template <typename... KArgs, typename... Args>
inline void launch_kernel(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t st, Args &&...args)
{
    static_assert(sizeof...(KArgs) == sizeof...(Args), "one argument per kernel parameter");
    std::tuple<KArgs...> vals(static_cast<KArgs>(std::forward<Args>(args))...);
    void *ptrs[sizeof...(KArgs) > 0 ? sizeof...(KArgs) : 1];
    launch_pointers(vals, ptrs, std::index_sequence_for<KArgs...>{});
    set_launch_status(hipLaunchKernel(reinterpret_cast<const void *>(kernel), grid, block, ptrs, lds, st));
}
#define HIPML_LAUNCH(kernel, grid, block, lds, st, ...) ::hipml::launch_kernel(kernel, grid, block, lds, st, __VA_ARGS__)

// The sigmoid output gate (crates/hipml-core/src/ops.rs:354-360): x / (1 + e^-g).  Every kernel that gates
// writes it through this one expression, so a fused call and the attention followed by the stand-alone
// gate kernel give the same bits.  The exponential is one v_exp_f32 of g * -log2(e) and the quotient one
// v_rcp_f32 (1 ulp each; ~3e-7 relative in all, inside the 1e-6 / 1e-5 the gate is held to against the
// CPU definition): the library expf and the IEEE division are ~20 instructions per value, which the
// chunk kernels pay on 32 values per lane with eight waves on a CU (2.3 us of a 672-token step).
// Large |g| saturate as the definition does (e^-g -> inf gives 0, -> 0 gives x).
__device__ __forceinline__ float gated(float x, float g)
{
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f));
}
#endif

inline hipStream_t as_stream(hipml_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// n_heads / n_kv / head_dim rules shared by the attention launchers
// (crates/hipml-kernels/src/launch_kv.rs:130-148 in the reference).
// (narrow: the decode launchers also take head_dim 64)
int check_heads(int n_heads, int n_kv, int head_dim, bool narrow = false);

// Kernel launchers implemented in the .hip translation units -------------------

struct RopeTable {
    const float *dev;  // [max_pos][n_rot/2][2] cos,sin or nullptr
    float theta;
    int n_rot;
    int max_pos;
    int device_angles; // opt-in: positions outside the table may use f64 pow/sincos on the device
};

int launch_mrope(hipStream_t st, const float *x, float *y, int n_heads, int head_dim, int n_rot,
                 int s0, int s1, int s2, int s3, const int32_t *pos, int pos_stride, int rows,
                 float theta, const RopeTable &tab);
int launch_rope_chunk(hipStream_t st, float *q, float *k, int n_head, int n_kv, int head_dim,
                      int n_rot, float theta, int pos0, int tokens, const RopeTable &tab);
int launch_kv_encode(hipStream_t st, int q4, const float *k, const float *v, uint8_t *kc, uint8_t *vc,
                     int n_kv, int head_dim, int stride, const int32_t *pos, int pos_stride,
                     size_t slot_bytes, int slots, int start, int src0, int rows);
// rope_chunk + kv_encode_bulk(start = pos0, src0 = 0, rows = tokens) in one launch (n_rot must be 64).
int launch_rope_encode_chunk(hipStream_t st, int q4, float *q, float *k, const float *v, uint8_t *kc,
                             uint8_t *vc, int n_head, int n_kv, int n_rot, float theta, int pos0,
                             int tokens, int stride, const RopeTable &tab);
int launch_kv_rows_copy(hipStream_t st, int q4, const uint8_t *k_src, const uint8_t *v_src, uint8_t *k_dst,
                        uint8_t *v_dst, int n_kv, int src_stride, int dst_stride, int rows);
int launch_front(hipStream_t st, const float *qg, float *q, float *gate, float *k, const float *qw,
                 const float *kw, int n_heads, int n_kv, int n_rot, int s0, int s1, int s2, int s3,
                 const int32_t *pos, int pos0, int rows, float theta, float eps, const RopeTable &tab,
                 int enc = -1, const float *v = nullptr, uint8_t *kc = nullptr, uint8_t *vc = nullptr,
                 const int32_t *step = nullptr, int start = 0, int stride = 0,
                 const int32_t *rowpos = nullptr, size_t slot_bytes = 0);
int launch_q_gate(hipStream_t st, const float *x, const float *gate, float *y, size_t n);

struct DecodeLaunch {
    const float *q;
    const uint8_t *k;
    const uint8_t *v;
    float *part_acc;
    float *part_ml;
    float *out;
    const float *gate;  // rows laid out like `out`, or nullptr: out *= sigmoid(gate) in the merge
    const int32_t *pos; // (pos, seq) pairs, one per row
    int n_heads, n_kv, stride, splits, slots;
    int head_dim; // 256: the MFMA kernels; 64: the plain fp32 kernels
    int q4; // cache format: 0 = q8_0, 1 = q4_0
    int exact; // q8_0 only: the fp32-class variant (Q and the weights as hi + lo f16 pairs)
    float scale;
    size_t kv_slot_bytes, acc_slot, ml_slot, q_slot;
    uint16_t row0[kMaxSlots]; // first row of each slot
    uint8_t cols[kMaxSlots];  // rows of each slot (1..kMaxCols)
    int total_rows;
    int max_cols;
};
int launch_decode_q8(hipStream_t st, const DecodeLaunch &a);
// Raise the decode kernels' dynamic LDS limit (once per device; called by hipml_attn_init).
int decode_init();
// Look up the current device's copy of the decode kernels' built-in scratch array (called by
// hipml_attn_init with `device` current), and hand it out as the partial buffers of one call.
int decode_static_init(int device);
int decode_static_partials(int n_heads, int splits, float **part_acc, float **part_ml);
// The process-wide choice between split + merge launches (0) and one launch whose workgroups merge their
// partials themselves (1) for a single sequence over q8_0; on < 0 only reads it.  Returns the old value.
int decode_one_launch(int on);

// Raise the prefill kernels' dynamic LDS limit (once per process; called by hipml_attn_init).
int prefill_init();
int launch_chunk_q8(hipStream_t st, const float *q, const uint8_t *kc, const uint8_t *vc,
                    float *out, int n_head, int n_kv, int pos0, int tokens, int stride,
                    float *part_acc, float *part_ml, int splits, const float *gate, int q4, void *out16 = nullptr,
                    const void *kv_f16 = nullptr, const float *rope_tab = nullptr);
// The f16 copy of a cache that launch_chunk_q8 can read instead of the cache (kv_f16): its size for
// `stride` rows per KV head, and the conversion of the 64-key tiles that hold rows [start, start + rows).
size_t kv_f16_bytes(int stride, int n_kv);
// The scratch slice count that lets a sliced chunk over the cache of `slices` slices run over f16 tiles made in
// the tail of its scratch (launch_chunk_q8 takes that path by itself when the count it is given allows it).
int chunk_tiles_splits(int pos0, int tokens, int n_head, int n_kv, int slices);
bool chunk_tiles_pay(int pos0, int tokens); // the shapes for which hipml_attn_chunk_splits asks for that count
int launch_kv_f16_rows(hipStream_t st, const uint8_t *kc, const uint8_t *vc, void *copy, int n_kv, int stride,
                       int start, int rows, int q4);

// y[r][row] = W[row][:] . x[r][:] over a Q8_0 weight matrix, rows <= 128 activation rows (proj.hip).
int launch_gemv_q8_rows(hipStream_t st, const uint8_t *w, const float *x, float *y, int m, int k, int rows);
// The same product for a prefill chunk: f16 operands on MFMA, fp32 accumulation (proj.hip).
// With a scratch of tokens*k f16 (x16) the activations are gated (gate may be null) and converted once
// by a first kernel; without it the GEMM converts the f32 activations itself (gate must be null).
int launch_gemm_q8_f16(hipStream_t st, const uint8_t *w, const float *x, const float *gate, float *y, int m,
                       int k, int tokens, void *x16);
// Raise the projection kernels' dynamic LDS limit (once per process; called by hipml_attn_init).
int proj_init();

// Measurement-only kernels (yardstick.hip): a pure read of two arrays in the decode kernel's access pattern
// (mode 0: global_load_lds, 1: register loads), and a loop of independent MFMAs on one wave per SIMD.
int yardstick_init();
int launch_bench_stream(hipStream_t st, const uint8_t *a, const uint8_t *b, size_t bytes_each, int mode, uint32_t *sink);
int launch_bench_mfma(hipStream_t st, int workgroups, int iters, float *sink, unsigned long long *clocks);

} // namespace hipml
