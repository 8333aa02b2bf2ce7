// C ABI of libhipml_attn.so: argument validation and launcher selection.
// Every entry point validates on the host, then launches asynchronously on the
// caller's stream; nothing here allocates, frees or synchronises.

#include "common.h"

#include <atomic>
#include <math.h>
#include <mutex>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

namespace hipml {

static thread_local char g_err[512] = "";
// The registered RoPE table is a device pointer, so there is one registration per device: the entry
// points that rotate work on a snapshot of the current device's, taken under the lock when they start
// (snapshot_rope), and the two calls that change it write under the same lock.
static RopeTable g_rope_dev[64];
static std::mutex g_rope_mu;
static thread_local RopeTable g_rope = {nullptr, 0.0f, 0, 0, 0};
static std::atomic<bool> g_inited[64]; // per device: hipml_attn_init has run with that device current

static int rope_device()
{
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64)
        device = 0;
    return device;
}

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

// Start of every entry point: no message.
void clear_error() { g_err[0] = '\0'; }

// Entry points that rotate work on a snapshot of the current device's RoPE registration.
static void snapshot_rope()
{
    const int device = rope_device();
    std::lock_guard<std::mutex> lock(g_rope_mu);
    g_rope = g_rope_dev[device];
}

static thread_local hipError_t g_launch_status = hipSuccess;
void set_launch_status(hipError_t e) { g_launch_status = e; }

int launched(const char *what)
{
    const hipError_t e = g_launch_status;
    if (e == hipSuccess)
        return 0;
    snprintf(g_err, sizeof(g_err), "%s launch failed: %d (%s)", what, (int)e, hipGetErrorString(e));
    return (int)e;
}

int check_heads(int n_heads, int n_kv, int head_dim, bool narrow)
{
    if (n_kv <= 0 || n_heads <= 0 || n_heads % n_kv != 0)
        return fail(HIPML_ATTN_E_SHAPE, "n_heads %d is not a multiple of n_kv %d", n_heads, n_kv);
    const int group = n_heads / n_kv;
    if (group > kMaxGroup)
        return fail(HIPML_ATTN_E_SHAPE, "GQA group %d > %d: one workgroup covers at most %d heads",
                    group, kMaxGroup, kMaxGroup);
    if (narrow && head_dim == 64)
        return 0;
    if (head_dim != kHeadDim)
        return fail(HIPML_ATTN_E_SHAPE, "head_dim %d: the gfx950 attention kernels are head_dim %d%s",
                    head_dim, kHeadDim, narrow ? " (decode also 64)" : " only");
    return 0;
}

// KV dtype ids of the reference's KvDtype::id (crates/hipml-core/src/kv.rs:47-91): 0 = q8_0, 1 = q4_0.
static int check_kv_dtype(int dtype)
{
    if (dtype == 0 || dtype == 1)
        return 0;
    return fail(HIPML_ATTN_E_UNSUPPORTED, "unknown KV dtype %d (0 = q8_0, 1 = q4_0)", dtype);
}

// Decode launchers: the reference's selector also names kernel variants
// (crates/hipml-kernels/src/launch_kv.rs:146-170,329-334): 0 and 4 are its q8_0 kernels as shipped,
// 1 and 5 the q4_0 ones, and 6 keeps its all-f32 staged q8_0 kernel reachable.  Here 0/4 run the
// q8_0 kernel with f16-class weights, 6 its fp32-class variant (Q and the weights as hi + lo f16
// pairs: the precision of the reference's f32 arithmetic), 1/5 the q4_0 kernel; the other values
// (A/B variants of the reference's own kernels) are refused.
// *kv_dtype: 0 = q8_0, 1 = q4_0, 2 = q8_0 fp32-class.
static int decode_format(int dtype, int *kv_dtype)
{
    if (dtype == 0 || dtype == 4) {
        *kv_dtype = 0;
        return 0;
    }
    if (dtype == 1 || dtype == 5) {
        *kv_dtype = 1;
        return 0;
    }
    if (dtype == 6) {
        *kv_dtype = 2;
        return 0;
    }
    return fail(HIPML_ATTN_E_UNSUPPORTED,
                "KV dtype selector %d: 0/4 (q8_0), 6 (q8_0, fp32-class) and 1/5 (q4_0) are built", dtype);
}

// The MFMA kernels keep more LDS than a launch may use by default; hipml_attn_init raises the limit
// on the device it is called for, so a launch needs that call for the device that is current now.
static int require_init()
{
    int device = -1;
    const hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess || device < 0 || device >= 64 || !g_inited[device])
        return fail(HIPML_ATTN_E_STATE, "hipml_attn_init has not been called for the current device (%d)",
                    e == hipSuccess ? device : -1);
    return 0;
}

static int check_aligned16(const void *p, const char *name)
{
    if (((uintptr_t)p & 15) != 0)
        return fail(HIPML_ATTN_E_RANGE, "%s must be 16-byte aligned", name);
    return 0;
}

#define REQUIRE_PTR(p)                                                                              \
    do {                                                                                            \
        if ((p) == nullptr)                                                                         \
            return fail(HIPML_ATTN_E_NULL, "%s is NULL", #p);                                        \
    } while (0)

// ---- f16 shadows of caches ------------------------------------------------------------------------
// A cache registered with hipml_kv_f16_attach has an f16 tile copy that this library keeps: every entry
// point that writes rows of the cache at positions the host knows converts those rows right behind its own
// launch, the ones whose positions live in device memory mark the shadow stale (the next chunk attention
// over the cache then converts every live row once), and the chunk attention over the cache reads the
// tiles instead of making them per call.  The bookkeeping is host state, updated when a call is issued
// (or captured), not when a captured graph is replayed.
struct KvShadow {
    const uint8_t *kc, *vc;
    void *copy;
    int n_kv, stride, q4;
    int valid;  // rows [0, valid) of the copy match the cache
    bool stale; // rows were written at positions only the device knows
};
constexpr int kMaxShadows = 1024;
static std::mutex g_shadow_mu;
static KvShadow g_shadows[kMaxShadows];
static int g_nshadows = 0;

static int shadow_index(const void *kc) // (lock held)
{
    for (int i = 0; i < g_nshadows; i++)
        if (g_shadows[i].kc == kc)
            return i;
    return -1;
}

// Rows [start, start + rows) of the cache at kc have been written by a launch already issued on st.
static int shadow_rows_written(hipStream_t st, const void *kc, int start, int rows)
{
    if (rows <= 0)
        return 0;
    KvShadow sh;
    {
        std::lock_guard<std::mutex> lock(g_shadow_mu);
        const int i = shadow_index(kc);
        if (i < 0)
            return 0;
        sh = g_shadows[i];
        if (sh.stale || start > sh.valid)
            return 0; // (the chunk attention converts from `valid` on, or everything, when it needs the rows)
        g_shadows[i].valid = sh.valid > start + rows ? sh.valid : start + rows;
    }
    return launch_kv_f16_rows(st, sh.kc, sh.vc, sh.copy, sh.n_kv, sh.stride, start, rows, sh.q4);
}

// Rows of the caches inside [base, base + bytes) have been written at positions only the device knows.
static void shadow_rows_unknown(const void *base, size_t bytes)
{
    std::lock_guard<std::mutex> lock(g_shadow_mu);
    const uint8_t *lo = static_cast<const uint8_t *>(base);
    for (int i = 0; i < g_nshadows; i++)
        if (g_shadows[i].kc >= lo && g_shadows[i].kc < lo + (bytes > 0 ? bytes : 1))
            g_shadows[i].stale = true;
}

// The shadow the chunk attention over (kc, vc) may read for rows [0, need), brought up to date on st;
// false: there is none (or it belongs to another geometry).
static bool shadow_for_chunk(hipStream_t st, const void *kc, const void *vc, int n_kv, int stride, int q4, int need,
                             const void **copy, int *rc)
{
    KvShadow sh;
    int from;
    {
        std::lock_guard<std::mutex> lock(g_shadow_mu);
        const int i = shadow_index(kc);
        if (i < 0 || g_shadows[i].vc != vc || g_shadows[i].n_kv != n_kv || g_shadows[i].stride != stride ||
            g_shadows[i].q4 != q4)
            return false;
        sh = g_shadows[i];
        from = sh.stale ? 0 : (sh.valid < need ? sh.valid : need);
        g_shadows[i].stale = false;
        g_shadows[i].valid = sh.stale || sh.valid < need ? need : sh.valid;
    }
    *copy = sh.copy;
    *rc = from < need ? launch_kv_f16_rows(st, sh.kc, sh.vc, sh.copy, sh.n_kv, sh.stride, from, need - from, sh.q4) : 0;
    return true;
}

static int decode_common(hipStream_t st, int dtype, const int32_t *pos, const float *q, const void *k,
                         const void *v, float *part_acc, float *part_ml, float *out, int n_heads,
                         int n_kv, int head_dim, int stride, float scale, int splits,
                         size_t kv_slot_bytes, size_t acc_slot, size_t ml_slot, size_t q_slot,
                         int slots, const int32_t *cols_per_slot, const float *gate = nullptr)
{
    REQUIRE_PTR(pos);
    REQUIRE_PTR(q);
    REQUIRE_PTR(k);
    REQUIRE_PTR(v);
    REQUIRE_PTR(part_acc);
    REQUIRE_PTR(part_ml);
    REQUIRE_PTR(out);
    int rc = check_heads(n_heads, n_kv, head_dim, true);
    if (rc)
        return rc;
    if (stride <= 0)
        return fail(HIPML_ATTN_E_RANGE, "stride %d must be positive", stride);
    if (splits < 1 || splits > 4096)
        return fail(HIPML_ATTN_E_RANGE, "splits %d outside 1..4096", splits);
    if (slots < 1 || slots > kMaxSlots)
        return fail(HIPML_ATTN_E_RANGE, "slots %d outside 1..%d", slots, kMaxSlots);
    if ((rc = check_aligned16(k, "k cache")) || (rc = check_aligned16(v, "v cache")) ||
        (rc = check_aligned16(q, "q")) || (rc = check_aligned16(part_acc, "part_acc")) ||
        (rc = check_aligned16(out, "out")) || (rc = check_aligned16(gate, "gate")))
        return rc;
    if (kv_slot_bytes % 16 != 0 || q_slot % 4 != 0 || acc_slot % 4 != 0)
        return fail(HIPML_ATTN_E_RANGE, "slot strides must keep 16-byte alignment");

    DecodeLaunch L;
    memset(&L, 0, sizeof(L));
    L.q = q;
    L.k = static_cast<const uint8_t *>(k);
    L.v = static_cast<const uint8_t *>(v);
    L.part_acc = part_acc;
    L.part_ml = part_ml;
    L.out = out;
    L.gate = gate;
    L.pos = pos;
    L.n_heads = n_heads;
    L.n_kv = n_kv;
    L.head_dim = head_dim;
    L.stride = stride;
    L.splits = splits;
    L.slots = slots;
    L.q4 = dtype == 1 ? 1 : 0;
    L.exact = dtype == 2 ? 1 : 0;
    L.scale = scale;
    L.kv_slot_bytes = kv_slot_bytes;
    L.acc_slot = acc_slot;
    L.ml_slot = ml_slot;
    L.q_slot = q_slot;
    int rows = 0, max_cols = 0;
    for (int s = 0; s < slots; s++) {
        const int c = cols_per_slot ? cols_per_slot[s] : 1;
        if (c < 1 || c > kMaxCols)
            return fail(HIPML_ATTN_E_RANGE, "slot %d carries %d query rows; 1..%d supported", s, c,
                        kMaxCols);
        L.row0[s] = (uint16_t)rows;
        L.cols[s] = (uint8_t)c;
        rows += c;
        max_cols = c > max_cols ? c : max_cols;
    }
    L.total_rows = rows;
    L.max_cols = max_cols;
    if ((rc = require_init()))
        return rc;
    return launch_decode_q8(st, L);
}

} // namespace hipml

using namespace hipml;

extern "C" {

int hipml_attn_init(int device)
{
    clear_error();
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess)
        return fail((int)e, "hipGetDeviceProperties(%d) failed: %d (%s)", device, (int)e,
                    hipGetErrorString(e));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(HIPML_ATTN_E_DEVICE, "device %d is %s; this library is built for gfx950 only",
                    device, prop.gcnArchName);
    if (device < 0 || device >= 64)
        return fail(HIPML_ATTN_E_RANGE, "device %d outside 0..63", device);
    // the per-kernel limits and the scratch symbol belong to the current device: make `device` current
    // for the set-up and put the caller's device back afterwards
    int before = -1;
    e = hipGetDevice(&before);
    if (e == hipSuccess && before != device)
        e = hipSetDevice(device);
    if (e != hipSuccess)
        return fail((int)e, "selecting device %d failed: %d (%s)", device, (int)e, hipGetErrorString(e));
    int rc = decode_init();
    if (rc == 0)
        rc = decode_static_init(device);
    if (rc == 0)
        rc = prefill_init();
    if (rc == 0)
        rc = proj_init();
    if (rc == 0)
        rc = yardstick_init();
    if (before != device)
        (void)hipSetDevice(before);
    if (rc)
        return rc;
    g_inited[device] = true;
    return 0;
}

const char *hipml_attn_last_error(void) { return g_err; }

const char *hipml_attn_version(void) { return "hipml-attn-mi355x 0.2 (gfx950)"; }

// ---- split policies -------------------------------------------------------------------

int hipml_attn_decode_splits(int seq, int n_kv)
{
    // One workgroup of four waves walks 32-key tiles; give every workgroup at least one tile per
    // wave (128 keys) and stop at two workgroups per CU (512) across the KV heads.  That is the scratch
    // the q4_0 kernel wants (depth 32,768: 20.4 us per layer with 128 splits, 23.5 with 64); over q8_0
    // the launch uses half of it, one workgroup per CU: the merge then reads half the partials, and the
    // rows stream no slower (19.2 us with 64 splits, 20.4 with 128; at 131,072: 51.9 against 52.5).
    if (seq < 1 || n_kv < 1)
        return 1;
    int by_work = (seq + 127) / 128;
    int by_cus = 512 / n_kv;
    if (by_cus < 1)
        by_cus = 1;
    int s = by_work < by_cus ? by_work : by_cus;
    return s < 1 ? 1 : s;
}

int hipml_attn_batch_splits(int stride, int n_kv, int slots)
{
    if (stride < 1 || n_kv < 1 || slots < 1)
        return 1;
    // Batches of up to a quarter of the chip's workgroup window in slots run as one window of workers
    // that share the slots by depth (see the decode kernel); `splits` is then only the cap on one
    // slot's workers and the width of its partials, and a generous cap lets a deep slot among
    // shallow ones take more of the chip (16 slots, one of depth 16,384 and fifteen of 512: 51 us at
    // cap 16, 37 us at cap 32).  Larger batches launch every split of every slot; there two windows
    // of workgroups were the best compromise between all-deep and skewed batches.
    int by_work = (stride + 127) / 128;
    const int window = 512 / n_kv;
    int by_cus = (4 * slots <= window ? 2048 : 1024) / (n_kv * slots);
    if (by_cus > 64)
        by_cus = 64;
    if (by_cus < 1)
        by_cus = 1;
    int s = by_work < by_cus ? by_work : by_cus;
    return s < 1 ? 1 : s;
}

int hipml_attn_chunk_slices(int pos0, int tokens, int n_kv)
{
    // A prefill workgroup is 8 tasks of (32 tokens x 1 head) and owns a whole CU (two 66 KiB LDS
    // buffers), and the hardware starts workgroups in rounds of as many as fit the chip (256).  A
    // launch of `splits` key slices is therefore priced as
    //     rounds x (key tiles of the longest slice + 4),   rounds = ceil(workgroups / 256),
    // the 4 tiles standing for what a workgroup costs whatever its slice (fetching and transposing its
    // Q rows, writing its partial rows), with the workgroups counted as the kernel cuts them (a task
    // block whose last token sees few key tiles gets fewer slices), and the cheapest slice count wins:
    // it is the one that fills its last round (672 tokens at depth 32,768: 4 slices = one full round,
    // 584 us, against 610 for the two rounds of 8; 256 tokens there: 10 slices = 240 workgroups, where
    // 12 would leave a second round of 32).  Slices keep at least 128 keys, and n_kv * splits is a
    // multiple of the 8 XCDs where that is possible (the kernel then keeps each slice's K/V stream
    // inside one XCD's L2).  Heads per KV head are taken as 6, the geometry built.
    if (tokens < 1 || n_kv < 1)
        return 1;
    const int group = 6, tasks_per_wg = 8, q_tile = 32, k_tile = 64;
    const int ntask = (tokens + q_tile - 1) / q_tile * group;
    const int nblock = (ntask + tasks_per_wg - 1) / tasks_per_wg;
    if (n_kv * nblock >= 512)
        return 1;
    const int keys = pos0 + tokens;
    const int by_work = keys / 128;
    const int tiles_last = (keys + k_tile - 1) / k_tile;
    int best = 1;
    double best_cost = 0.0;
    for (int pass = 0; pass < 2; pass++) { // first the slice counts that suit the XCDs, then any
        for (int s = 1; s <= 16 && s <= (by_work > 1 ? by_work : 1); s++) {
            if (pass == 0 && s > 1 && (n_kv * s) % 8 != 0)
                continue;
            const int slice_tiles = (tiles_last + s - 1) / s;
            long wg = 0;
            for (int tb = 0; tb < nblock; tb++) {
                const int last_task = tb * tasks_per_wg + tasks_per_wg - 1 < ntask ? tb * tasks_per_wg + tasks_per_wg - 1
                                                                                 : ntask - 1;
                const int tt_last = last_task / group;
                const int last_tok = ((tt_last + 1) * q_tile < tokens ? (tt_last + 1) * q_tile : tokens) - 1;
                const int tiles_b = (pos0 + last_tok + 1 + k_tile - 1) / k_tile;
                const int n = (tiles_b + slice_tiles - 1) / slice_tiles;
                wg += n < 1 ? 1 : (n < s ? n : s);
            }
            wg *= n_kv;
            const long rounds = (wg + 255) / 256;
            const double cost = (double)rounds * (slice_tiles + 4.0);
            if (best_cost == 0.0 || cost < best_cost) {
                best = s;
                best_cost = cost;
            }
        }
        if (best > 1)
            break;
    }
    return best;
}

int hipml_attn_chunk_splits(int pos0, int tokens, int n_kv)
{
    // 0 = the kernel that keeps the key slices inside the workgroup (no partial rows in memory, no merge
    // launch).  Its workgroups share the dequantized K/V among two heads instead of eight tasks, so it
    // pays where the rows (Q, gate, output, partial rows) outweigh the keys: chunks near position 0.
    // Measured against the best slice count of the other kernel, whole step in us (this one first):
    // 32 @ 0 16.7 / 20.6, 128 @ 0 18.5 / 26.4, 256 @ 0 24.8 / 35.1, 672 @ 0 41.7 / 52.1, 1,024 @ 0 61.6 / 66.8,
    // 1,536 @ 0 101 / 113, 2,048 @ 0 150 / 149, 4,096 @ 0 428 / 416; 128 @ 256 27.2 / 31.4, 256 @ 512 38.0 /
    // 37.8, 672 @ 512 54.1 / 58.2, 1,024 @ 512 84.3 / 103, 672 @ 1,024 68.7 / 68.0, 256 @ 1,024 48.9 / 43.6,
    // 64 @ 1,000 45.4 / 34.5, 672 @ 8,192 293 / 200.
    if (tokens >= 1 && n_kv >= 1 && pos0 >= 0 && (long long)pos0 + tokens <= 1792 && pos0 <= 2 * tokens)
        return 0;
    const int slices = hipml_attn_chunk_slices(pos0, tokens, n_kv);
    // Long chunks behind a prefix at least as long: a scratch sized for this many slices also holds the live rows as f16 tiles,
    // and the call then runs `slices` slices of the 64-token kernel over those (2,048 @ 100,000: 13 for 4
    // slices, 4.1 against 4.7 ms).  Heads per KV head are taken as 6, as in hipml_attn_chunk_slices.
    if (slices >= 2 && chunk_tiles_pay(pos0, tokens)) {
        const int with_tiles = chunk_tiles_splits(pos0, tokens, 6 * n_kv, n_kv, slices);
        if (with_tiles <= 64)
            return with_tiles;
    }
    return slices;
}

// ---- RoPE ----------------------------------------------------------------------------------

size_t hipml_rope_table_bytes(int n_rot, int max_pos)
{
    if (n_rot <= 0 || (n_rot & 1) || max_pos <= 0)
        return 0;
    return (size_t)max_pos * (size_t)(n_rot / 2) * 2 * sizeof(float);
}

int hipml_rope_table_fill_host(float *host_table, float theta_base, int n_rot, int max_pos)
{
    clear_error();
    REQUIRE_PTR(host_table);
    if (n_rot <= 0 || (n_rot & 1) || max_pos <= 0)
        return fail(HIPML_ATTN_E_RANGE, "n_rot %d must be even and positive, max_pos %d positive",
                    n_rot, max_pos);
    const int half = n_rot / 2;
    for (int k = 0; k < half; k++) {
        // same expression, same libm, as the CPU definition (ops.rs:296-300 of the reference)
        const double freq = pow((double)theta_base, -2.0 * (double)k / (double)n_rot);
        for (int p = 0; p < max_pos; p++) {
            const double ang = (double)p * freq;
            float *e = host_table + ((size_t)p * half + k) * 2;
            e[0] = (float)cos(ang);
            e[1] = (float)sin(ang);
        }
    }
    return 0;
}

int hipml_rope_set_table(const float *dev_table, float theta_base, int n_rot, int max_pos)
{
    clear_error();
    if (dev_table != nullptr && (n_rot <= 0 || (n_rot & 1) || max_pos <= 0))
        return fail(HIPML_ATTN_E_RANGE, "n_rot %d must be even and positive, max_pos %d positive",
                    n_rot, max_pos);
    const int device = rope_device();
    std::lock_guard<std::mutex> lock(g_rope_mu);
    RopeTable &t = g_rope_dev[device];
    t.dev = dev_table;
    t.theta = theta_base;
    t.n_rot = n_rot;
    t.max_pos = dev_table ? max_pos : 0;
    return 0;
}

int hipml_rope_allow_device_angles(int allow)
{
    clear_error();
    const int device = rope_device();
    std::lock_guard<std::mutex> lock(g_rope_mu);
    g_rope_dev[device].device_angles = allow ? 1 : 0;
    return 0;
}

// Positions pos0 .. pos0 + tokens - 1 known to the host: all inside the table, unless the caller has
// opted in to device angles.
static int check_rope_range(int pos0, int tokens)
{
    if (!g_rope.device_angles && tokens > 0 && (long long)pos0 + tokens > g_rope.max_pos)
        return fail(HIPML_ATTN_E_RANGE,
                    "positions %d..%lld lie outside the RoPE table of %d rows (register n_ctx rows with "
                    "hipml_rope_set_table, or opt in with hipml_rope_allow_device_angles)",
                    pos0, (long long)pos0 + tokens - 1, g_rope.max_pos);
    return 0;
}

static int check_rope(int n_heads, int head_dim, int n_rot, float theta)
{
    if (n_heads <= 0 || head_dim <= 0)
        return fail(HIPML_ATTN_E_SHAPE, "n_heads %d / head_dim %d must be positive", n_heads,
                    head_dim);
    if (n_rot <= 0 || (n_rot & 1) || n_rot > head_dim)
        return fail(HIPML_ATTN_E_SHAPE, "n_rot %d must be even and <= head_dim %d", n_rot, head_dim);
    if (g_rope.dev == nullptr || g_rope.theta != theta || g_rope.n_rot != n_rot)
        return fail(HIPML_ATTN_E_STATE,
                    "no RoPE table registered for theta %g n_rot %d (hipml_rope_set_table)", theta,
                    n_rot);
    return 0;
}

int hipml_mrope_f32(hipml_stream_t stream, const float *x, float *y, int n_heads, int head_dim,
                    int n_rot, int s0, int s1, int s2, int s3, const int32_t *pos,
                    float theta_base)
{
    clear_error();
    snapshot_rope();
    REQUIRE_PTR(x);
    REQUIRE_PTR(y);
    REQUIRE_PTR(pos);
    int rc = check_rope(n_heads, head_dim, n_rot, theta_base);
    if (rc)
        return rc;
    if (s0 < 0 || s1 < 0 || s2 < 0 || s3 < 0)
        return fail(HIPML_ATTN_E_RANGE, "negative M-RoPE section");
    return launch_mrope(as_stream(stream), x, y, n_heads, head_dim, n_rot, s0, s1, s2, s3, pos, 0,
                        1, theta_base, g_rope);
}

int hipml_mrope_rows_f32(hipml_stream_t stream, const float *x, float *y, int n_heads,
                         int head_dim, int n_rot, int s0, int s1, int s2, int s3,
                         const int32_t *pos, int rows, float theta_base)
{
    clear_error();
    snapshot_rope();
    REQUIRE_PTR(x);
    REQUIRE_PTR(y);
    REQUIRE_PTR(pos);
    int rc = check_rope(n_heads, head_dim, n_rot, theta_base);
    if (rc)
        return rc;
    if (rows < 0)
        return fail(HIPML_ATTN_E_RANGE, "rows %d is negative", rows);
    if (rows == 0)
        return 0;
    return launch_mrope(as_stream(stream), x, y, n_heads, head_dim, n_rot, s0, s1, s2, s3, pos, 2,
                        rows, theta_base, g_rope);
}

int hipml_rope_chunk_f32(hipml_stream_t stream, float *q, float *k, int n_head, int n_kv,
                         int head_dim, int n_rot, float theta_base, int pos0, int tokens)
{
    clear_error();
    snapshot_rope();
    REQUIRE_PTR(q);
    REQUIRE_PTR(k);
    int rc = check_rope(n_head, head_dim, n_rot, theta_base);
    if (rc)
        return rc;
    if (n_kv <= 0)
        return fail(HIPML_ATTN_E_SHAPE, "n_kv %d must be positive", n_kv);
    if (pos0 < 0 || tokens < 0)
        return fail(HIPML_ATTN_E_RANGE, "pos0 %d / tokens %d must be non-negative", pos0, tokens);
    if ((rc = check_rope_range(pos0, tokens)))
        return rc;
    if (tokens == 0)
        return 0;
    return launch_rope_chunk(as_stream(stream), q, k, n_head, n_kv, head_dim, n_rot, theta_base,
                             pos0, tokens, g_rope);
}

// ---- attention front end ---------------------------------------------------------------------

static int check_front(const float *qg, const float *q, const float *gate, const float *k,
                       const float *q_norm, const float *k_norm, int n_heads, int n_kv, int head_dim,
                       int n_rot, float theta_base, float eps)
{
    if (qg == nullptr || q == nullptr || gate == nullptr || k == nullptr || q_norm == nullptr ||
        k_norm == nullptr)
        return fail(HIPML_ATTN_E_NULL, "a front-end buffer (qg, q, gate, k, q_norm, k_norm) is NULL");
    int rc = check_rope(n_heads, head_dim, n_rot, theta_base);
    if (rc)
        return rc;
    if (n_kv <= 0)
        return fail(HIPML_ATTN_E_SHAPE, "n_kv %d must be positive", n_kv);
    if (head_dim != kHeadDim)
        return fail(HIPML_ATTN_E_UNSUPPORTED,
                    "attention front end: built for head_dim %d (one square per lane slot and the "
                    "256-wide tree of the reference), got %d", kHeadDim, head_dim);
    if (!(eps >= 0.0f))
        return fail(HIPML_ATTN_E_RANGE, "eps %g must be non-negative", (double)eps);
    return 0;
}

int hipml_attn_front_f32(hipml_stream_t stream, const float *qg, float *q, float *gate, float *k,
                         const float *q_norm, const float *k_norm, int n_heads, int n_kv,
                         int head_dim, int n_rot, int s0, int s1, int s2, int s3,
                         const int32_t *pos, float theta_base, float eps)
{
    clear_error();
    snapshot_rope();
    REQUIRE_PTR(pos);
    int rc = check_front(qg, q, gate, k, q_norm, k_norm, n_heads, n_kv, head_dim, n_rot, theta_base, eps);
    if (rc)
        return rc;
    if (s0 < 0 || s1 < 0 || s2 < 0 || s3 < 0)
        return fail(HIPML_ATTN_E_RANGE, "negative M-RoPE section");
    return launch_front(as_stream(stream), qg, q, gate, k, q_norm, k_norm, n_heads, n_kv, n_rot, s0, s1,
                        s2, s3, pos, 0, 1, theta_base, eps, g_rope);
}

int hipml_attn_chunk_front_f32(hipml_stream_t stream, const float *qg, float *k, float *q,
                               float *gate, const float *q_norm, const float *k_norm, int n_heads,
                               int n_kv, int head_dim, int n_rot, float theta_base, float eps,
                               int pos0, int tokens)
{
    clear_error();
    snapshot_rope();
    int rc = check_front(qg, q, gate, k, q_norm, k_norm, n_heads, n_kv, head_dim, n_rot, theta_base, eps);
    if (rc)
        return rc;
    if (pos0 < 0 || tokens < 0)
        return fail(HIPML_ATTN_E_RANGE, "pos0 %d / tokens %d must be non-negative", pos0, tokens);
    if ((rc = check_rope_range(pos0, tokens)))
        return rc;
    if (tokens == 0)
        return 0;
    return launch_front(as_stream(stream), qg, q, gate, k, q_norm, k_norm, n_heads, n_kv, n_rot, 0, 0, 0,
                        0, nullptr, pos0, tokens, theta_base, eps, g_rope);
}

// ---- KV append -------------------------------------------------------------------------------

static int check_encode(int dtype, const void *k, const void *v, const void *kc, const void *vc,
                        int n_kv, int head_dim, int stride)
{
    int rc = check_kv_dtype(dtype);
    if (rc)
        return rc;
    if (k == nullptr || v == nullptr || kc == nullptr || vc == nullptr)
        return fail(HIPML_ATTN_E_NULL, "a K/V source or cache pointer is NULL");
    if (n_kv <= 0)
        return fail(HIPML_ATTN_E_SHAPE, "n_kv %d must be positive", n_kv);
    if (head_dim <= 0 || head_dim % 32 != 0 || head_dim > 256)
        return fail(HIPML_ATTN_E_SHAPE, "head_dim %d: must be 32..=256, multiple of 32", head_dim);
    if (stride <= 0)
        return fail(HIPML_ATTN_E_RANGE, "stride %d must be positive", stride);
    return 0;
}

// The front end and the append of the finished K row and of the V row in one launch.
int hipml_attn_front_encode_f32(hipml_stream_t stream, const int32_t *step, int dtype, const float *qg,
                                float *q, float *gate, float *k, const float *v, const float *q_norm,
                                const float *k_norm, void *k_cache, void *v_cache, int n_heads, int n_kv,
                                int head_dim, int n_rot, int s0, int s1, int s2, int s3, float theta_base,
                                float eps, int stride)
{
    clear_error();
    snapshot_rope();
    REQUIRE_PTR(step);
    int rc = check_front(qg, q, gate, k, q_norm, k_norm, n_heads, n_kv, head_dim, n_rot, theta_base, eps);
    if (rc == 0)
        rc = check_encode(dtype, k, v, k_cache, v_cache, n_kv, head_dim, stride);
    if (rc)
        return rc;
    if (s0 < 0 || s1 < 0 || s2 < 0 || s3 < 0)
        return fail(HIPML_ATTN_E_RANGE, "negative M-RoPE section");
    shadow_rows_unknown(k_cache, 1);
    return launch_front(as_stream(stream), qg, q, gate, k, q_norm, k_norm, n_heads, n_kv, n_rot, s0, s1,
                        s2, s3, step + 4, 0, 1, theta_base, eps, g_rope, dtype, v,
                        static_cast<uint8_t *>(k_cache), static_cast<uint8_t *>(v_cache), step, 0, stride);
}

int hipml_attn_chunk_front_encode_f32(hipml_stream_t stream, int dtype, const float *qg, float *k,
                                      const float *v, float *q, float *gate, const float *q_norm,
                                      const float *k_norm, void *k_cache, void *v_cache, int n_heads,
                                      int n_kv, int head_dim, int n_rot, float theta_base, float eps,
                                      int pos0, int tokens, int stride)
{
    clear_error();
    snapshot_rope();
    int rc = check_front(qg, q, gate, k, q_norm, k_norm, n_heads, n_kv, head_dim, n_rot, theta_base, eps);
    if (rc == 0)
        rc = check_encode(dtype, k, v, k_cache, v_cache, n_kv, head_dim, stride);
    if (rc)
        return rc;
    if (pos0 < 0 || tokens < 0)
        return fail(HIPML_ATTN_E_RANGE, "pos0 %d / tokens %d must be non-negative", pos0, tokens);
    if ((rc = check_rope_range(pos0, tokens)))
        return rc;
    if ((long long)pos0 + tokens > stride)
        return fail(HIPML_ATTN_E_RANGE, "rows [%d, %d) do not fit a cache of %d rows per head", pos0,
                    pos0 + tokens, stride);
    if (tokens == 0)
        return 0;
    rc = launch_front(as_stream(stream), qg, q, gate, k, q_norm, k_norm, n_heads, n_kv, n_rot, 0, 0, 0,
                      0, nullptr, pos0, tokens, theta_base, eps, g_rope, dtype, v,
                      static_cast<uint8_t *>(k_cache), static_cast<uint8_t *>(v_cache), nullptr, pos0,
                      stride);
    return rc ? rc : shadow_rows_written(as_stream(stream), k_cache, pos0, tokens);
}

// The batched engine's front end: row r belongs to sequence r and rotates at text position pos[2 r].
int hipml_attn_front_rows_f32(hipml_stream_t stream, const float *qg, float *k, float *q, float *gate,
                              const float *q_norm, const float *k_norm, int n_heads, int n_kv,
                              int head_dim, int n_rot, float theta_base, float eps, const int32_t *pos,
                              int rows)
{
    clear_error();
    snapshot_rope();
    REQUIRE_PTR(pos);
    int rc = check_front(qg, q, gate, k, q_norm, k_norm, n_heads, n_kv, head_dim, n_rot, theta_base, eps);
    if (rc)
        return rc;
    if (rows < 0)
        return fail(HIPML_ATTN_E_RANGE, "rows %d is negative", rows);
    if (rows == 0)
        return 0;
    return launch_front(as_stream(stream), qg, q, gate, k, q_norm, k_norm, n_heads, n_kv, n_rot, 0, 0, 0,
                        0, nullptr, 0, rows, theta_base, eps, g_rope, -1, nullptr, nullptr, nullptr, nullptr,
                        0, 0, pos, 0);
}

// The same with the append of every row's K and V into its sequence's cache (slot r starts
// r * slot_bytes into the caches), at position pos[2 r].
int hipml_attn_front_rows_encode_f32(hipml_stream_t stream, int dtype, const float *qg, float *k,
                                     const float *v, float *q, float *gate, const float *q_norm,
                                     const float *k_norm, void *k_cache, void *v_cache, int n_heads,
                                     int n_kv, int head_dim, int n_rot, float theta_base, float eps,
                                     int stride, const int32_t *pos, size_t slot_bytes, int slots)
{
    clear_error();
    snapshot_rope();
    REQUIRE_PTR(pos);
    int rc = check_front(qg, q, gate, k, q_norm, k_norm, n_heads, n_kv, head_dim, n_rot, theta_base, eps);
    if (rc == 0)
        rc = check_encode(dtype, k, v, k_cache, v_cache, n_kv, head_dim, stride);
    if (rc)
        return rc;
    if (slots < 0)
        return fail(HIPML_ATTN_E_RANGE, "slots %d is negative", slots);
    if (slots == 0)
        return 0;
    shadow_rows_unknown(k_cache, slot_bytes * (size_t)slots);
    return launch_front(as_stream(stream), qg, q, gate, k, q_norm, k_norm, n_heads, n_kv, n_rot, 0, 0, 0,
                        0, nullptr, 0, slots, theta_base, eps, g_rope, dtype, v,
                        static_cast<uint8_t *>(k_cache), static_cast<uint8_t *>(v_cache), nullptr, 0, stride,
                        pos, slot_bytes);
}

int hipml_kv_encode(hipml_stream_t stream, const int32_t *step, int dtype, const float *k_in,
                    const float *v_in, void *k_cache, void *v_cache, int n_kv, int head_dim,
                    int stride)
{
    clear_error();
    REQUIRE_PTR(step);
    int rc = check_encode(dtype, k_in, v_in, k_cache, v_cache, n_kv, head_dim, stride);
    if (rc)
        return rc;
    shadow_rows_unknown(k_cache, 1);
    return launch_kv_encode(as_stream(stream), dtype, k_in, v_in, static_cast<uint8_t *>(k_cache),
                               static_cast<uint8_t *>(v_cache), n_kv, head_dim, stride, step, 0, 0,
                               1, 0, 0, 1);
}

int hipml_kv_encode_bulk(hipml_stream_t stream, int dtype, const float *k_f32, const float *v_f32,
                         void *k_cache, void *v_cache, int n_kv, int head_dim, int stride,
                         int start, int src0, int rows)
{
    clear_error();
    int rc = check_encode(dtype, k_f32, v_f32, k_cache, v_cache, n_kv, head_dim, stride);
    if (rc)
        return rc;
    if (start < 0 || src0 < 0 || rows < 0)
        return fail(HIPML_ATTN_E_RANGE, "start %d / src0 %d / rows %d must be non-negative", start,
                    src0, rows);
    if ((long long)start + rows > stride)
        return fail(HIPML_ATTN_E_RANGE, "rows [%d, %d) do not fit a cache of %d rows per head",
                    start, start + rows, stride);
    rc = launch_kv_encode(as_stream(stream), dtype, k_f32, v_f32, static_cast<uint8_t *>(k_cache),
                          static_cast<uint8_t *>(v_cache), n_kv, head_dim, stride, nullptr, 0,
                          0, rows, start, src0, rows);
    return rc ? rc : shadow_rows_written(as_stream(stream), k_cache, start, rows);
}

int hipml_rope_encode_chunk_f32(hipml_stream_t stream, float *q, float *k, const float *v, void *k_cache,
                                void *v_cache, int n_head, int n_kv, int head_dim, int n_rot,
                                float theta_base, int pos0, int tokens, int dtype, int stride)
{
    clear_error();
    snapshot_rope();
    // (q may be NULL: only the K rows are rotated, for a caller whose attention call rotates the query rows)
    int rc = check_rope(n_head, head_dim, n_rot, theta_base);
    if (rc == 0)
        rc = check_encode(dtype, k, v, k_cache, v_cache, n_kv, head_dim, stride);
    if (rc)
        return rc;
    if (head_dim != kHeadDim || n_rot != 64)
        return fail(HIPML_ATTN_E_UNSUPPORTED, "head_dim %d / n_rot %d: the fused kernel is built for %d / 64",
                    head_dim, n_rot, kHeadDim);
    if (pos0 < 0 || tokens < 0)
        return fail(HIPML_ATTN_E_RANGE, "pos0 %d / tokens %d must be non-negative", pos0, tokens);
    if ((rc = check_rope_range(pos0, tokens)))
        return rc;
    if ((long long)pos0 + tokens > stride)
        return fail(HIPML_ATTN_E_RANGE, "rows [%d, %d) do not fit a cache of %d rows per head", pos0,
                    pos0 + tokens, stride);
    if (tokens == 0)
        return 0;
    rc = launch_rope_encode_chunk(as_stream(stream), dtype, q, k, v, static_cast<uint8_t *>(k_cache),
                                  static_cast<uint8_t *>(v_cache), n_head, n_kv, n_rot, theta_base, pos0,
                                  tokens, stride, g_rope);
    return rc ? rc : shadow_rows_written(as_stream(stream), k_cache, pos0, tokens);
}

int hipml_kv_encode_rows(hipml_stream_t stream, int dtype, const float *k_f32, const float *v_f32,
                         void *k_cache, void *v_cache, int n_kv, int head_dim, int stride,
                         const int32_t *pos, size_t slot_bytes, int slots)
{
    clear_error();
    REQUIRE_PTR(pos);
    int rc = check_encode(dtype, k_f32, v_f32, k_cache, v_cache, n_kv, head_dim, stride);
    if (rc)
        return rc;
    if (slots < 0)
        return fail(HIPML_ATTN_E_RANGE, "slots %d is negative", slots);
    shadow_rows_unknown(k_cache, slot_bytes * (size_t)(slots > 0 ? slots : 0));
    return launch_kv_encode(as_stream(stream), dtype, k_f32, v_f32, static_cast<uint8_t *>(k_cache),
                               static_cast<uint8_t *>(v_cache), n_kv, head_dim, stride, pos, 2,
                               slot_bytes, slots, 0, 0, slots);
}

int hipml_kv_rows_copy(hipml_stream_t stream, int dtype, const void *k_src, const void *v_src, void *k_dst,
                       void *v_dst, int n_kv, int head_dim, int src_stride, int dst_stride, int rows)
{
    clear_error();
    int rc = check_kv_dtype(dtype);
    if (rc)
        return rc;
    REQUIRE_PTR(k_src);
    REQUIRE_PTR(v_src);
    REQUIRE_PTR(k_dst);
    REQUIRE_PTR(v_dst);
    if (head_dim != kHeadDim)
        return fail(HIPML_ATTN_E_UNSUPPORTED, "head_dim %d: this library is built for %d", head_dim, kHeadDim);
    if (n_kv < 1 || n_kv > 64)
        return fail(HIPML_ATTN_E_RANGE, "n_kv %d outside 1..64", n_kv);
    if (rows < 0 || rows > src_stride || rows > dst_stride)
        return fail(HIPML_ATTN_E_RANGE, "rows %d do not fit strides %d -> %d", rows, src_stride, dst_stride);
    if ((rc = check_aligned16(k_src, "k_src")) || (rc = check_aligned16(v_src, "v_src")) ||
        (rc = check_aligned16(k_dst, "k_dst")) || (rc = check_aligned16(v_dst, "v_dst")))
        return rc;
    rc = launch_kv_rows_copy(as_stream(stream), dtype, static_cast<const uint8_t *>(k_src),
                             static_cast<const uint8_t *>(v_src), static_cast<uint8_t *>(k_dst),
                             static_cast<uint8_t *>(v_dst), n_kv, src_stride, dst_stride, rows);
    return rc ? rc : shadow_rows_written(as_stream(stream), k_dst, 0, rows);
}

// ---- decode ------------------------------------------------------------------------------------

int hipml_attn_decode_kv(hipml_stream_t stream, const int32_t *step, int dtype, const float *q,
                         const void *k, const void *v, float *part_acc, float *part_ml,
                         float *out, int n_heads, int n_kv, int head_dim, int stride, float scale,
                         int splits, size_t k_off, size_t v_off)
{
    clear_error();
    int fmt = 0;
    int rc = decode_format(dtype, &fmt);
    if (rc)
        return rc;
    REQUIRE_PTR(k);
    REQUIRE_PTR(v);
    const size_t slice = (size_t)(n_heads > 0 ? n_heads : 0) * (size_t)(splits > 0 ? splits : 0);
    return decode_common(as_stream(stream), fmt, step, q, static_cast<const uint8_t *>(k) + k_off,
                         static_cast<const uint8_t *>(v) + v_off, part_acc, part_ml, out, n_heads,
                         n_kv, head_dim, stride, scale, splits, 0, slice * (size_t)(head_dim > 0 ? head_dim : 0), slice * 2,
                         (size_t)n_heads * (size_t)(head_dim > 0 ? head_dim : 0), 1, nullptr);
}

int hipml_attn_decode_kv_noalloc(hipml_stream_t stream, const int32_t *step, int dtype, const float *q,
                                 const void *k, const void *v, float *out, int n_heads, int n_kv,
                                 int head_dim, int stride, float scale, int splits, size_t k_off,
                                 size_t v_off)
{
    clear_error();
    int rc = check_heads(n_heads, n_kv, head_dim);
    if (rc)
        return rc;
    float *part_acc = nullptr, *part_ml = nullptr;
    if ((rc = decode_static_partials(n_heads, splits, &part_acc, &part_ml)))
        return rc;
    return hipml_attn_decode_kv(stream, step, dtype, q, k, v, part_acc, part_ml, out, n_heads, n_kv,
                                head_dim, stride, scale, splits, k_off, v_off);
}

int hipml_attn_decode_one_launch(int on) { return decode_one_launch(on); }

int hipml_attn_decode_kv_cols(hipml_stream_t stream, int dtype, const int32_t *pos,
                              const float *q, const void *k, const void *v, float *part_acc,
                              float *part_ml, float *out, int n_heads, int n_kv, int head_dim,
                              int stride, float scale, int splits, int cols, size_t acc_slot,
                              size_t ml_slot, size_t q_slot)
{
    clear_error();
    int fmt = 0;
    int rc = decode_format(dtype, &fmt);
    if (rc)
        return rc;
    if (cols < 1 || cols > kMaxCols)
        return fail(HIPML_ATTN_E_RANGE, "cols %d outside 1..%d", cols, kMaxCols);
    const int32_t one_slot[1] = {cols};
    return decode_common(as_stream(stream), fmt, pos, q, k, v, part_acc, part_ml, out, n_heads, n_kv,
                         head_dim, stride, scale, splits, 0, acc_slot, ml_slot, q_slot, 1,
                         one_slot);
}

int hipml_attn_decode_rows(hipml_stream_t stream, int dtype, const int32_t *pos, const float *q,
                           const void *k_cache, const void *v_cache, float *part_acc,
                           float *part_ml, float *out, int n_heads, int n_kv, int head_dim,
                           int stride, float scale, int splits, size_t kv_slot_bytes,
                           size_t acc_slot, size_t ml_slot, size_t q_slot, int slots)
{
    clear_error();
    int fmt = 0;
    int rc = decode_format(dtype, &fmt);
    if (rc)
        return rc;
    if (slots < 1 || slots > kMaxSlots)
        return fail(HIPML_ATTN_E_RANGE, "slots %d outside 1..%d", slots, kMaxSlots);
    if (kv_slot_bytes == 0 && slots <= kMaxCols && slots > 1) {
        // rows of one sequence sharing a cache: stream it once for all of them
        const int32_t one_slot[1] = {slots};
        return decode_common(as_stream(stream), fmt, pos, q, k_cache, v_cache, part_acc, part_ml, out,
                             n_heads, n_kv, head_dim, stride, scale, splits, 0, acc_slot, ml_slot,
                             q_slot, 1, one_slot);
    }
    return decode_common(as_stream(stream), fmt, pos, q, k_cache, v_cache, part_acc, part_ml, out,
                         n_heads, n_kv, head_dim, stride, scale, splits, kv_slot_bytes, acc_slot,
                         ml_slot, q_slot, slots, nullptr);
}

int hipml_attn_decode_batch(hipml_stream_t stream, int dtype, const int32_t *pos, const float *q,
                            const void *k_cache, const void *v_cache, float *part_acc,
                            float *part_ml, float *out, int n_heads, int n_kv, int head_dim,
                            int stride, float scale, int splits, size_t kv_slot_bytes,
                            size_t acc_slot, size_t ml_slot, size_t q_slot, int slots,
                            int live_seq)
{
    clear_error();
    if (live_seq < 0 || live_seq > stride)
        return fail(HIPML_ATTN_E_RANGE, "live_seq %d outside 0..stride %d", live_seq, stride);
    return hipml_attn_decode_rows(stream, dtype, pos, q, k_cache, v_cache, part_acc, part_ml, out,
                                  n_heads, n_kv, head_dim, stride, scale, splits, kv_slot_bytes,
                                  acc_slot, ml_slot, q_slot, slots);
}

int hipml_attn_decode_batch_cols(hipml_stream_t stream, int dtype, const int32_t *pos,
                                 const float *q, const void *k_cache, const void *v_cache,
                                 float *part_acc, float *part_ml, float *out, int n_heads,
                                 int n_kv, int head_dim, int stride, float scale, int splits,
                                 size_t kv_slot_bytes, size_t acc_slot, size_t ml_slot,
                                 size_t q_slot, int slots, const int32_t *cols_per_slot_host)
{
    clear_error();
    int fmt = 0;
    int rc = decode_format(dtype, &fmt);
    if (rc)
        return rc;
    REQUIRE_PTR(cols_per_slot_host);
    return decode_common(as_stream(stream), fmt, pos, q, k_cache, v_cache, part_acc, part_ml, out,
                         n_heads, n_kv, head_dim, stride, scale, splits, kv_slot_bytes, acc_slot,
                         ml_slot, q_slot, slots, cols_per_slot_host);
}

int hipml_attn_decode_kv_gate(hipml_stream_t stream, const int32_t *step, int dtype, const float *q,
                              const void *k, const void *v, float *part_acc, float *part_ml,
                              float *out, const float *gate, int n_heads, int n_kv, int head_dim,
                              int stride, float scale, int splits, size_t k_off, size_t v_off)
{
    clear_error();
    int fmt = 0;
    int rc = decode_format(dtype, &fmt);
    if (rc)
        return rc;
    REQUIRE_PTR(k);
    REQUIRE_PTR(v);
    REQUIRE_PTR(gate);
    const size_t slice = (size_t)(n_heads > 0 ? n_heads : 0) * (size_t)(splits > 0 ? splits : 0);
    return decode_common(as_stream(stream), fmt, step, q, static_cast<const uint8_t *>(k) + k_off,
                         static_cast<const uint8_t *>(v) + v_off, part_acc, part_ml, out, n_heads,
                         n_kv, head_dim, stride, scale, splits, 0, slice * (size_t)(head_dim > 0 ? head_dim : 0), slice * 2,
                         (size_t)n_heads * (size_t)(head_dim > 0 ? head_dim : 0), 1, nullptr, gate);
}

int hipml_attn_decode_batch_cols_gate(hipml_stream_t stream, int dtype, const int32_t *pos,
                                      const float *q, const void *k_cache, const void *v_cache,
                                      float *part_acc, float *part_ml, float *out,
                                      const float *gate, int n_heads, int n_kv, int head_dim,
                                      int stride, float scale, int splits, size_t kv_slot_bytes,
                                      size_t acc_slot, size_t ml_slot, size_t q_slot, int slots,
                                      const int32_t *cols_per_slot_host)
{
    clear_error();
    int fmt = 0;
    int rc = decode_format(dtype, &fmt);
    if (rc)
        return rc;
    REQUIRE_PTR(cols_per_slot_host);
    REQUIRE_PTR(gate);
    return decode_common(as_stream(stream), fmt, pos, q, k_cache, v_cache, part_acc, part_ml, out,
                         n_heads, n_kv, head_dim, stride, scale, splits, kv_slot_bytes, acc_slot,
                         ml_slot, q_slot, slots, cols_per_slot_host, gate);
}

// ---- chunk prefill ---------------------------------------------------------------------------------

// Everything chunk_q8_common can refuse, without a launch: the entry point that rotates q in place first
// runs these checks before it touches q.
static int chunk_q8_validate(const float *q, const void *kc, const void *vc, float *out, const float *gate,
                             bool want_gate, int n_head, int n_kv, int head_dim, int pos0, int tokens, int dtype,
                             int stride, float *part_acc, float *part_ml, int splits, void *out16, bool want_f16)
{
    REQUIRE_PTR(q);
    REQUIRE_PTR(kc);
    REQUIRE_PTR(vc);
    REQUIRE_PTR(out);
    if (want_f16) {
        REQUIRE_PTR(out16);
        if (int rc16 = check_aligned16(out16, "out16"))
            return rc16;
    }
    if (want_gate)
        REQUIRE_PTR(gate);
    // the reference's chunk launcher numbers the formats 1 = q8_0, 2 = q4_0
    // (crates/hipml-kernels/src/attn_gpu/imp/attn_chunk_kv.rs:41-60)
    if (dtype != 1 && dtype != 2)
        return fail(HIPML_ATTN_E_UNSUPPORTED,
                    "quantized chunk attention: dtype 1 (q8_0) or 2 (q4_0), got %d", dtype);
    int rc = check_heads(n_head, n_kv, head_dim);
    if (rc)
        return rc;
    if (pos0 < 0 || tokens < 0)
        return fail(HIPML_ATTN_E_RANGE, "pos0 %d / tokens %d must be non-negative", pos0, tokens);
    if ((long long)pos0 + tokens > stride)
        return fail(HIPML_ATTN_E_RANGE, "chunk [%d, %d) does not fit a cache of %d rows per head",
                    pos0, pos0 + tokens, stride);
    if (splits > 64)
        return fail(HIPML_ATTN_E_RANGE, "splits %d > 64", splits);
    if (splits >= 2) {
        REQUIRE_PTR(part_acc);
        REQUIRE_PTR(part_ml);
    }
    if ((rc = check_aligned16(q, "q")) || (rc = check_aligned16(out, "out")) ||
        (rc = check_aligned16(kc, "k cache")) || (rc = check_aligned16(vc, "v cache")))
        return rc;
    if (want_gate && (rc = check_aligned16(gate, "gate")))
        return rc;
    return tokens == 0 ? 0 : require_init();
}

static int chunk_q8_common(hipml_stream_t stream, const float *q, const void *kc, const void *vc,
                           float *out, const float *gate, bool want_gate, int n_head, int n_kv,
                           int head_dim, int pos0, int tokens, int dtype, int stride, float *part_acc,
                           float *part_ml, int splits, void *out16 = nullptr, bool want_f16 = false,
                           const void *kv_f16 = nullptr, const float *rope_tab = nullptr)
{
    clear_error();
    int rc = chunk_q8_validate(q, kc, vc, out, gate, want_gate, n_head, n_kv, head_dim, pos0, tokens, dtype, stride,
                               part_acc, part_ml, splits, out16, want_f16);
    if (rc || tokens == 0)
        return rc;
    // a cache with a registered f16 shadow: the sliced attention reads its tiles (as many slices as the policy
    // gives a chunk over such a copy, within what the scratch was sized for)
    if (splits >= 2 && kv_f16 == nullptr && rope_tab == nullptr) {
        const void *copy = nullptr;
        if (shadow_for_chunk(as_stream(stream), kc, vc, n_kv, stride, dtype == 2 ? 1 : 0, pos0 + tokens, &copy, &rc)) {
            if (rc)
                return rc;
            const int slices = hipml_attn_chunk_slices(pos0, tokens, n_kv);
            kv_f16 = copy;
            splits = slices < splits ? (slices < 1 ? 1 : slices) : splits;
            dtype = 1; // (the tiles are f16 whatever the cache holds)
        }
    }
    return launch_chunk_q8(as_stream(stream), q, static_cast<const uint8_t *>(kc),
                           static_cast<const uint8_t *>(vc), out, n_head, n_kv, pos0, tokens,
                           stride, part_acc, part_ml, splits, want_gate ? gate : nullptr, dtype == 2 ? 1 : 0,
                           want_f16 ? out16 : nullptr, kv_f16, rope_tab);
}

int hipml_attn_chunk_q8_split(hipml_stream_t stream, const float *q, const void *kc,
                              const void *vc, float *out, int n_head, int n_kv, int head_dim,
                              int pos0, int tokens, int dtype, int stride, float *part_acc,
                              float *part_ml, int splits)
{
    return chunk_q8_common(stream, q, kc, vc, out, nullptr, false, n_head, n_kv, head_dim, pos0, tokens,
                           dtype, stride, part_acc, part_ml, splits);
}

int hipml_attn_chunk_q8_split_gate(hipml_stream_t stream, const float *q, const void *kc,
                                   const void *vc, const float *gate, float *out, int n_head,
                                   int n_kv, int head_dim, int pos0, int tokens, int dtype,
                                   int stride, float *part_acc, float *part_ml, int splits)
{
    return chunk_q8_common(stream, q, kc, vc, out, gate, true, n_head, n_kv, head_dim, pos0, tokens,
                           dtype, stride, part_acc, part_ml, splits);
}

int hipml_attn_chunk_q8_split_gate_f16(hipml_stream_t stream, const float *q, const void *kc,
                                       const void *vc, const float *gate, float *out, void *out16,
                                       int n_head, int n_kv, int head_dim, int pos0, int tokens, int dtype,
                                       int stride, float *part_acc, float *part_ml, int splits)
{
    return chunk_q8_common(stream, q, kc, vc, out, gate, true, n_head, n_kv, head_dim, pos0, tokens,
                           dtype, stride, part_acc, part_ml, splits, out16, true);
}

int hipml_attn_chunk_rope_q8(hipml_stream_t stream, float *q, const void *kc, const void *vc, const float *gate,
                             float *out, void *out16, int n_head, int n_kv, int head_dim, int n_rot,
                             float theta_base, int pos0, int tokens, int dtype, int stride, float *part_acc,
                             float *part_ml, int splits)
{
    clear_error();
    snapshot_rope();
    REQUIRE_PTR(q);
    int rc = check_rope(n_head, head_dim, n_rot, theta_base);
    if (rc)
        return rc;
    if (pos0 < 0 || tokens < 0)
        return fail(HIPML_ATTN_E_RANGE, "pos0 %d / tokens %d must be non-negative", pos0, tokens);
    if ((rc = check_rope_range(pos0, tokens)))
        return rc;
    // The in-workgroup kernel rotates the rows where it loads them (table positions only); any other
    // kernel gets them rotated in place first.
    const bool in_kernel = splits == 0 && n_rot == 64 && head_dim == kHeadDim &&
                           (long long)pos0 + tokens <= g_rope.max_pos;
    // nothing may be refused once q has been rotated in place: a corrected retry would rotate it again
    if ((rc = chunk_q8_validate(q, kc, vc, out, gate, gate != nullptr, n_head, n_kv, head_dim, pos0, tokens, dtype,
                                stride, part_acc, part_ml, splits, out16, out16 != nullptr)))
        return rc;
    if (!in_kernel && tokens > 0) {
        if ((rc = check_aligned16(q, "q")))
            return rc;
        if ((rc = require_init()))
            return rc;
        if ((rc = launch_rope_chunk(as_stream(stream), q, q, n_head, 0, head_dim, n_rot, theta_base, pos0, tokens,
                                    g_rope)))
            return rc;
    }
    return chunk_q8_common(stream, q, kc, vc, out, gate, gate != nullptr, n_head, n_kv, head_dim, pos0, tokens,
                           dtype, stride, part_acc, part_ml, splits, out16, out16 != nullptr, nullptr,
                           in_kernel ? g_rope.dev : nullptr);
}

// ---- chunk prefill over the f16 copy of a cache ----------------------------------------------------

size_t hipml_kv_f16_bytes(int stride, int n_kv)
{
    if (stride < 1 || n_kv < 1)
        return 0;
    return kv_f16_bytes(stride, n_kv);
}

int hipml_kv_f16_rows(hipml_stream_t stream, int dtype, const void *k_cache, const void *v_cache,
                      void *kv_f16, int n_kv, int head_dim, int stride, int start, int rows)
{
    clear_error();
    REQUIRE_PTR(k_cache);
    REQUIRE_PTR(v_cache);
    REQUIRE_PTR(kv_f16);
    if (dtype != 0 && dtype != 1)
        return fail(HIPML_ATTN_E_UNSUPPORTED, "KV dtype %d: 0 (q8_0) and 1 (q4_0) are built", dtype);
    if (head_dim != kHeadDim)
        return fail(HIPML_ATTN_E_UNSUPPORTED, "head_dim %d: the kernels are built for %d", head_dim, kHeadDim);
    if (n_kv < 1 || stride < 1)
        return fail(HIPML_ATTN_E_RANGE, "n_kv %d / stride %d must be positive", n_kv, stride);
    if (start < 0 || rows < 0 || (long long)start + rows > stride)
        return fail(HIPML_ATTN_E_RANGE, "rows [%d, %d + %d) do not fit a cache of %d rows per head", start,
                    start, rows, stride);
    int rc;
    if ((rc = check_aligned16(k_cache, "k cache")) || (rc = check_aligned16(v_cache, "v cache")) ||
        (rc = check_aligned16(kv_f16, "kv_f16")))
        return rc;
    if (rows == 0)
        return 0;
    if ((rc = require_init()))
        return rc;
    return launch_kv_f16_rows(as_stream(stream), static_cast<const uint8_t *>(k_cache),
                              static_cast<const uint8_t *>(v_cache), kv_f16, n_kv, stride, start, rows, dtype);
}

int hipml_kv_f16_attach(hipml_stream_t stream, int dtype, const void *k_cache, const void *v_cache, void *kv_f16,
                        int n_kv, int head_dim, int stride, int rows)
{
    // (the checks and the conversion of the rows the cache holds already)
    int rc = hipml_kv_f16_rows(stream, dtype, k_cache, v_cache, kv_f16, n_kv, head_dim, stride, 0, rows);
    if (rc)
        return rc;
    std::lock_guard<std::mutex> lock(g_shadow_mu);
    int i = shadow_index(k_cache);
    if (i < 0) {
        if (g_nshadows == kMaxShadows)
            return fail(HIPML_ATTN_E_RANGE, "%d caches have an f16 shadow already", kMaxShadows);
        i = g_nshadows++;
    }
    g_shadows[i] = KvShadow{static_cast<const uint8_t *>(k_cache), static_cast<const uint8_t *>(v_cache), kv_f16,
                            n_kv, stride, dtype, rows, false};
    return 0;
}

int hipml_kv_f16_detach(const void *k_cache)
{
    clear_error();
    std::lock_guard<std::mutex> lock(g_shadow_mu);
    const int i = shadow_index(k_cache);
    if (i < 0)
        return fail(HIPML_ATTN_E_STATE, "no f16 shadow is registered for this cache");
    g_shadows[i] = g_shadows[--g_nshadows];
    return 0;
}

int hipml_attn_chunk_kv_f16(hipml_stream_t stream, const float *q, const void *kv_f16, const float *gate,
                            float *out, void *out16, int n_head, int n_kv, int head_dim, int pos0, int tokens,
                            int stride, float *part_acc, float *part_ml, int splits)
{
    clear_error();
    REQUIRE_PTR(kv_f16);
    return chunk_q8_common(stream, q, kv_f16, kv_f16, out, gate, gate != nullptr, n_head, n_kv, head_dim, pos0,
                           tokens, 1, stride, part_acc, part_ml, splits, out16, out16 != nullptr, kv_f16);
}

// ---- gate ---------------------------------------------------------------------------------------------

int hipml_q_gate_f32(hipml_stream_t stream, const float *x, const float *gate, float *y, size_t n)
{
    clear_error();
    REQUIRE_PTR(x);
    REQUIRE_PTR(gate);
    REQUIRE_PTR(y);
    return launch_q_gate(as_stream(stream), x, gate, y, n);
}

// ---- projections over Q8_0 weights ----------------------------------------------------------------

int hipml_gemv_q8_0_rows(hipml_stream_t stream, const void *w, const float *x, float *y, int m, int k,
                         int rows)
{
    clear_error();
    REQUIRE_PTR(w);
    REQUIRE_PTR(x);
    REQUIRE_PTR(y);
    if (m < 1)
        return fail(HIPML_ATTN_E_RANGE, "m %d must be positive", m);
    if (k < 64 || k % 64 != 0)
        return fail(HIPML_ATTN_E_RANGE, "k %d must be a positive multiple of 64 (two Q8_0 blocks: rows "
                                        "stay dword aligned)", k);
    if (rows < 1 || rows > 128)
        return fail(HIPML_ATTN_E_RANGE, "rows %d outside 1..128", rows);
    if (((uintptr_t)w & 3) != 0)
        return fail(HIPML_ATTN_E_RANGE, "w must be 4-byte aligned");
    int rc = check_aligned16(x, "x");
    if (rc == 0)
        rc = require_init();
    if (rc)
        return rc;
    return launch_gemv_q8_rows(as_stream(stream), static_cast<const uint8_t *>(w), x, y, m, k, rows);
}

static int check_gemm(const void *w, const float *x, const float *y, int m, int k, int tokens)
{
    REQUIRE_PTR(w);
    REQUIRE_PTR(x);
    REQUIRE_PTR(y);
    if (m < 1)
        return fail(HIPML_ATTN_E_RANGE, "m %d must be positive", m);
    if (k < 64 || k % 64 != 0)
        return fail(HIPML_ATTN_E_RANGE, "k %d must be a positive multiple of 64 (two Q8_0 blocks: rows "
                                        "stay dword aligned)", k);
    if (tokens < 1)
        return fail(HIPML_ATTN_E_RANGE, "tokens %d must be positive", tokens);
    if (((uintptr_t)w & 3) != 0)
        return fail(HIPML_ATTN_E_RANGE, "w must be 4-byte aligned");
    int rc = check_aligned16(x, "x");
    return rc ? rc : require_init();
}

int hipml_gemm_q8_0_f16(hipml_stream_t stream, const void *w, const float *x, float *y, int m, int k,
                        int tokens)
{
    clear_error();
    int rc = check_gemm(w, x, y, m, k, tokens);
    if (rc)
        return rc;
    return launch_gemm_q8_f16(as_stream(stream), static_cast<const uint8_t *>(w), x, nullptr, y, m, k,
                              tokens, nullptr);
}

int hipml_attn_output_chunk_q8_0(hipml_stream_t stream, const void *wo, const float *attn_out,
                                 const float *gate, float *y, int m, int k, int tokens, void *x16)
{
    clear_error();
    REQUIRE_PTR(x16);
    // attn_out == NULL: x16 already holds the rows (hipml_attn_chunk_q8_split_gate_f16 wrote them)
    int rc = check_gemm(wo, attn_out ? attn_out : static_cast<const float *>(x16), y, m, k, tokens);
    if (rc)
        return rc;
    if (attn_out == nullptr && gate != nullptr)
        return fail(HIPML_ATTN_E_NULL, "a gate needs the f32 rows it applies to (attn_out is NULL)");
    if ((rc = check_aligned16(gate, "gate")) || (rc = check_aligned16(x16, "x16")))
        return rc;
    return launch_gemm_q8_f16(as_stream(stream), static_cast<const uint8_t *>(wo), attn_out, gate, y, m, k,
                              tokens, x16);
}

// ---- measurement only --------------------------------------------------------------------------

int hipml_bench_stream_read(hipml_stream_t stream, const void *a, const void *b, size_t bytes_each, int mode,
                            void *sink)
{
    clear_error();
    REQUIRE_PTR(a);
    REQUIRE_PTR(b);
    REQUIRE_PTR(sink);
    if (mode != 0 && mode != 1)
        return fail(HIPML_ATTN_E_RANGE, "mode %d: 0 (global memory to LDS) or 1 (register loads)", mode);
    if (bytes_each == 0 || bytes_each % (32 * kRowBytes) != 0 || bytes_each / (32 * kRowBytes) > 0x7fffffffu)
        return fail(HIPML_ATTN_E_RANGE, "bytes_each %zu must be a positive multiple of %d", bytes_each, 32 * kRowBytes);
    int rc;
    if ((rc = check_aligned16(a, "a")) || (rc = check_aligned16(b, "b")) || (rc = require_init()))
        return rc;
    return launch_bench_stream(as_stream(stream), static_cast<const uint8_t *>(a), static_cast<const uint8_t *>(b),
                               bytes_each, mode, static_cast<uint32_t *>(sink));
}

int hipml_bench_mfma_f16(hipml_stream_t stream, int workgroups, int iters, void *sink, void *clocks)
{
    clear_error();
    REQUIRE_PTR(sink);
    if (workgroups < 1 || workgroups > (1 << 20) || iters < 1)
        return fail(HIPML_ATTN_E_RANGE, "workgroups %d / iters %d out of range", workgroups, iters);
    if (((uintptr_t)clocks & 7) != 0)
        return fail(HIPML_ATTN_E_RANGE, "clocks must be 8-byte aligned");
    int rc = require_init();
    if (rc)
        return rc;
    return launch_bench_mfma(as_stream(stream), workgroups, iters, static_cast<float *>(sink),
                             static_cast<unsigned long long *>(clocks));
}

} // extern "C"
