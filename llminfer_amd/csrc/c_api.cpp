// C ABI of libllmi_hip.so: argument validation, the context-length dispatch,
// the hipMalloc-backed default pool and the copy helpers. The kernels live in
// mha_decode.hip and qk_norm_rope.hip.

#include <cstdint>
#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>

#include "llmi_hip.h"
#include "llmi_internal.h"
#include "pool.h"

namespace llmi {

namespace {
thread_local std::string g_last_error;

// Context lengths up to this run as one workgroup per KV head; longer ones are
// split over the 256 CUs. (The reference's threshold is 128 with 32-position
// splits, mha_kernel.cu:507-517. Here the split path pays three dependent
// memory round trips for its combine, while one workgroup streams a whole KV
// head of 11 tiles in about 4.4 us: measured at 32 query / 8 KV heads under graph
// replay, single pass against 8 splits 4.28 : 4.37 us at 160 positions, 4.41 : 4.45 at 176,
// 4.53 : 4.43 at 192, 4.73 : 4.53 at 208, 5.09 : 4.36 at 256.)
constexpr int kSinglePassMaxLen = 176;
// Workgroups the split path aims for: one per CU (256 CUs). Each workgroup keeps
// waves x stages x 8 KiB of loads in flight on its own; more, smaller splits only
// add partial-result traffic and lengthen the combine (measured, ctx 1K..32K).
constexpr int kTargetGroups = 256;
constexpr int kMinGroups = 128;
constexpr int kTile = 16;

inline int pow2_ceil(int x) {
    int p = 1;
    while (p < x) p <<= 1;
    return p;
}
inline int pow2_floor(int x) {
    int p = 1;
    while (p * 2 <= x) p <<= 1;
    return p;
}
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Tuning overrides from the environment, read once per process (the reference's counterparts are the compile-time
// constants of its dispatcher, mha_kernel.cu:478,505-517): LLMI_HIP_SINGLE_PASS_MAX = longest context that still runs
// as a single pass, LLMI_HIP_NUM_SPLITS = split count of the split path. Both apply only where the caller left the
// choice to the dispatcher (force_path AUTO / num_splits 0); anything unparsable or out of range is ignored.
struct EnvTuning {
    int single_pass_max = -1;  // -1: not set
    int num_splits = 0;        // 0: not set
};
int env_int(const char* name, long lo, long hi, int unset) {
    const char* v = std::getenv(name);
    if (!v || !*v) return unset;
    char* end = nullptr;
    const long x = std::strtol(v, &end, 10);
    if (!end || *end != '\0' || x < lo || x > hi) return unset;
    return (int)x;
}
const EnvTuning& env_tuning() {
    static const EnvTuning t = [] {
        EnvTuning e;
        e.single_pass_max = env_int("LLMI_HIP_SINGLE_PASS_MAX", 0, 1 << 20, -1);
        e.num_splits = env_int("LLMI_HIP_NUM_SPLITS", 2, kMaxSplits, 0);
        return e;
    }();
    return t;
}
}  // namespace

int record_hip_error(hipError_t err, const char* what) {
    if (err == hipSuccess) return LLMI_OK;
    g_last_error = std::string(what) + ": " + hipGetErrorString(err);
    return LLMI_ERR_LAUNCH;
}

unsigned long long next_epoch() {
    // Starts from the clock so that a stale record left in a reused workspace by another process
    // does not match. record_tag() turns it into a tag that is never zero.
    static std::atomic<unsigned long long> counter{
        (unsigned long long)std::chrono::steady_clock::now().time_since_epoch().count()};
    return counter.fetch_add(1, std::memory_order_relaxed);
}

// Default: far beyond any real kernel time (seconds), yet finite. LLMI_HIP_POLL_LIMIT in the environment replaces the
// default (read once, when the library is loaded); llmi_hip_set_poll_limit changes it at run time.
static int default_poll_limit() {
    const char* v = std::getenv("LLMI_HIP_POLL_LIMIT");
    if (v && *v) {
        char* end = nullptr;
        const long x = std::strtol(v, &end, 10);
        if (end && *end == '\0' && x >= 0 && x <= INT32_MAX) return (int)x;
    }
    return 1 << 22;
}
static std::atomic<int> g_poll_limit{default_poll_limit()};
int poll_limit() { return g_poll_limit.load(std::memory_order_relaxed); }
static std::atomic<int> g_test_far_home{0};
int test_far_home() { return g_test_far_home.load(std::memory_order_relaxed); }

// With 32 splits and more (16 for groups of eight query heads) the merge of a KV head's query heads is spread over as
// many workgroups; with fewer, the workgroup of the last split merges them all. Measured, 32 Q / 8 KV heads, spread
// against not: 16 splits 5.08 : 4.98 us at 1024 positions, 5.87 : 5.77 at 2048; 8 splits 4.51 : 4.41 at 256; 32 splits
// 5.03 : 5.14 at 1024, 5.71 : 5.80 at 2048, 6.86 : 7.08 at 4096, 7.88 : 8.10 at 6000; 64 Q heads, 16 splits 5.55 : 5.68 at
// 1024, 7.63 : 7.81 at 4096, 32 splits at 32768 24.4 : 25.3. LLMI_HIP_SPREAD_MIN_SPLITS moves the boundary.
int spread_merge_min_splits(int group_pad) {
    static const int v = env_int("LLMI_HIP_SPREAD_MIN_SPLITS", 1, 1 << 20, 0);
    return v ? v : group_pad >= 8 ? 16 : 32;
}

// Where the splits' runs start a multiple of 512 KiB apart, the workgroups of a KV head, walking in step, keep hitting
// the same few memory channels; the splits then start their walks at different tiles (STAGGER kernels, split s rotated
// by s & mask tiles of each wavefront's sequence).
// Position-major, runs up to 1 MiB, mask 3. 32 Q / 8 KV heads, with : without: 9.44 : 10.54 us at 8192 positions
// (512 KiB apart), level at 16384 (1 MiB); everywhere else the wrap-round only costs: 8.32 : 7.99 at 6144, 26.1 : 25.2
// at 32768, 47.6 : 45.5 at 65536, level at 2048, 4096, 7168, 9216 ... 24576.
// Head-major, runs of 512 KiB up to (not including) 2 MiB at a multiple of 512 KiB (up to 8 tiles above one count too:
// the position moves on by one per token), mask 31. With : without, two seconds of continuous replays each, 64 Q / 8 KV
// heads: 131072 positions (runs of 1 MiB) 80.0 : 86.3 us in the arena a fresh process allocates and 79.0 : 80.2 in
// another one, 32 Q heads 79.2 : 85.3 and 78.9 : 79.3; 196608 (1.5 MiB) 118.2 : 121.8; 65536 (512 KiB) 42.15 : 42.6 and
// 41.75 : 42.0. Not between the multiples (163840: 105.6 : 99.7; 98304: 63.8 : 63.35; 81920: 52.9 : 52.2), not from
// 2 MiB on (262144: 158.7 : 156.9), not below (32768: 23.27 : 22.63; 40960: 28.5 : 28.2). LLMI_HIP_STAGGER_MASK overrides
// the head-major mask (0 = never).
static int stagger_mask_override() {
    static const int v = env_int("LLMI_HIP_STAGGER_MASK", 0, 255, -1);
    return v;
}

int stagger_mask(int kv_layout, int64_t run_bytes, bool ragged) {
    if (kv_layout == LLMI_KV_LAYOUT_POS_MAJOR)
        return !ragged && run_bytes > 0 && run_bytes % (512 << 10) == 0 && run_bytes <= (1 << 20) ? 3 : 0;
    const int v = stagger_mask_override();
    if (v >= 0) return v;
    return head_major_stagger_rule(run_bytes);
}

// Position read on the device, head-major: the walk's kernels whenever the longest possible run reaches the rule's
// range (kStaggerByDevice: the kernel decides by the length it finds), the environment's mask as it is, else 0.
int dyn_stagger(int kv_layout, int64_t max_run_bytes) {
    if (kv_layout == LLMI_KV_LAYOUT_POS_MAJOR) return 0;
    const int v = stagger_mask_override();
    if (v >= 0) return v;
    return max_run_bytes >= (512 << 10) ? kStaggerByDevice : 0;
}

int check_launch() { return record_hip_error(hipGetLastError(), "kernel launch"); }

static int validate_mha(const llmi_mha_args* a) {
    if (!a) return LLMI_ERR_NULL_POINTER;
    if (!a->query || !a->key_cache || !a->value_cache || !a->output) return LLMI_ERR_NULL_POINTER;
    if (a->head_dim != 128) return LLMI_ERR_HEAD_DIM;                               // mha_kernel.cu:478-479
    if (a->kv_dim <= 0 || a->kv_dim % a->head_dim != 0) return LLMI_ERR_KV_DIM;     // mha_kernel.cu:494
    if (a->kv_mul < 1 || a->kv_mul > kMaxGroup) return LLMI_ERR_HEAD_GROUP;
    if (a->head_num != a->kv_mul * (a->kv_dim / a->head_dim)) return LLMI_ERR_HEAD_GROUP;
    if (a->max_seq_len <= 0 || a->layer_id < 0) return LLMI_ERR_INVALID_ARG;
    if (a->pos < 0 || a->pos >= a->max_seq_len) return LLMI_ERR_POS_RANGE;          // mha_kernel.cu:473-474
    if (a->kv_layout != LLMI_KV_LAYOUT_POS_MAJOR && a->kv_layout != LLMI_KV_LAYOUT_HEAD_MAJOR)
        return LLMI_ERR_LAYOUT;
    if (!aligned16(a->query) || !aligned16(a->key_cache) || !aligned16(a->value_cache) || !aligned16(a->output))
        return LLMI_ERR_ALIGNMENT;                                                  // mha_kernel.cu:495-498
    if (a->workspace && !aligned16(a->workspace)) return LLMI_ERR_ALIGNMENT;
    if (a->output_f32 && (reinterpret_cast<uintptr_t>(a->output_f32) & 3u)) return LLMI_ERR_ALIGNMENT;
    if (a->pos_device && (reinterpret_cast<uintptr_t>(a->pos_device) & 3u)) return LLMI_ERR_ALIGNMENT;
    if (a->force_path < LLMI_PATH_AUTO || a->force_path > LLMI_PATH_SPLIT_FUSED) return LLMI_ERR_INVALID_ARG;
    if (a->num_splits < 0 || a->num_splits > kMaxSplits) return LLMI_ERR_INVALID_ARG;
    const int w = a->waves_per_group;
    if (!(w == 0 || w == 1 || w == 2 || w == 4 || w == 8)) return LLMI_ERR_INVALID_ARG;
    return LLMI_OK;
}

// `wave_cap`: most wavefronts per workgroup the caller's kernel variant supports.
// `new_rows`: positions at the end of 0..pos that the kernel takes from registers instead of streaming
// them from the cache (1 in the append variant): the plan covers the others.
static int make_plan(const llmi_mha_args* a, llmi_mha_plan* p, int wave_cap = kMaxWaves, int new_rows = 0) {
    if (int rc = validate_mha(a)) return rc;
    const int seq_len = a->pos + 1 - new_rows;
    const int tiles = seq_len > 0 ? ceil_div(seq_len, kTile) : 1;  // (nothing cached yet: one workgroup all the same)
    const int n_kv = a->kv_dim / a->head_dim;
    const int group_pad = pow2_ceil(a->kv_mul);
    int max_waves = pow2_floor(kMaxGroupWaves / group_pad);
    if (max_waves > kMaxWaves) max_waves = kMaxWaves;
    if (a->waves_per_group > max_waves) return LLMI_ERR_INVALID_ARG;
    const size_t per_split_plain = (size_t)a->head_num * (a->head_dim + 2) * sizeof(float);
    // fused combine: per head and split, 128 partial outputs and two 8-byte arrival records
    const size_t per_split_fused = (size_t)a->head_num * (a->head_dim * sizeof(float) + 2 * sizeof(unsigned long long));

    const int single_waves_max = (max_waves < wave_cap ? max_waves : wave_cap);  // 8 where the kernel variant allows
    // Groups of 8 query heads run 8 waves per workgroup, which carry a single pass a little further
    // (64 query / 8 KV heads: single pass 5.14 us against 5.64 us split at 208 positions; at 256, where
    // 16 splits have a tile each, 5.51 against 5.34).
    int single_pass_max = (group_pad == 8 && wave_cap >= 8) ? 240 : kSinglePassMaxLen;
    if (env_tuning().single_pass_max >= 0) single_pass_max = env_tuning().single_pass_max;
    int path = a->force_path;
    if (path == LLMI_PATH_AUTO) {
        if (a->num_splits == 1) path = LLMI_PATH_SINGLE_PASS;
        else if (a->num_splits > 1) path = LLMI_PATH_SPLIT;
        else path = seq_len <= single_pass_max ? LLMI_PATH_SINGLE_PASS : LLMI_PATH_SPLIT_FUSED;
        if (path == LLMI_PATH_SPLIT) path = LLMI_PATH_SPLIT_FUSED;
    }
    // The separate combine kernel takes its split count from the launch, not from the device.
    if (a->pos_device && path == LLMI_PATH_SPLIT) return LLMI_ERR_INVALID_ARG;

    int num_splits = 1, tiles_per_split = tiles, waves;
    if (path != LLMI_PATH_SINGLE_PASS) {
        const bool fused = path == LLMI_PATH_SPLIT_FUSED;
        // Four waves per workgroup; eight for groups of 8 query heads, where the wider
        // merge pays (measured at 64 Q / 8 KV heads, ctx 4K..128K).
        int auto_waves = (group_pad == 8 && wave_cap >= 8) ? 8 : 4;
        if (auto_waves > max_waves) auto_waves = max_waves;
        waves = a->waves_per_group ? a->waves_per_group : auto_waves;
        int want = a->num_splits;
        const size_t per_split = fused ? per_split_fused : per_split_plain;
        const size_t cap = (a->workspace && a->workspace_bytes > 16) ? (a->workspace_bytes - 16) / per_split : 0;
        if (want == 0 && a->force_path == LLMI_PATH_AUTO && env_tuning().num_splits) {
            // the environment's split count, within what the caller's workspace holds
            if (cap < 2) return LLMI_ERR_WORKSPACE;
            want = env_tuning().num_splits;
            if ((size_t)want > cap) want = (int)cap;
        }
        if (want == 0) {
            // Auto: one workgroup per CU (kTargetGroups / kv heads splits) once half as many would need more
            // than a tile per wavefront; half as many below that, a quarter when even those would be left
            // without a tile. Measured with 32 query / 8 KV heads: 32 splits against 16 is 5.23 : 5.28 us
            // at 700 positions, 5.77 : 5.84 at 1500, 6.70 : 6.76 at 3000, 7.25 : 7.41 at 4096 and within
            // 1.5 % the other way at 512, 1024 and 2048. More, smaller splits only add partial-result
            // traffic and lengthen the combine (64 splits: +1 us everywhere).
            // And no more splits than the caller's workspace can hold.
            int target = kTargetGroups / n_kv;
            if (target < 2) target = 2;
            if (target > kMaxSplits) target = kMaxSplits;
            int half = kMinGroups / n_kv;
            if (half < 2) half = 2;
            int quarter = half / 2;
            if (quarter < 2) quarter = 2;
            // One workgroup per CU pays as soon as half as many splits would hold more than four tiles each (more than
            // one per wavefront at four wavefronts). Measured with the merge of a KV head's query heads spread over
            // several workgroups (which needs 32 splits to pay at groups of four, see spread_merge_min_splits), 32 Q / 8 KV
            // heads, head-major, 16 against 32 splits: 4.98 : 5.03 us at 1024 positions, 5.43 : 5.16 at 1200, 5.51 : 5.44 at
            // 1500, 5.69 : 5.60 at 1800, 5.77 : 5.71 at 2048, 6.49 : 6.40 at 3000, 7.16 : 6.86 at 4096; position-major 4.96 : 5.07
            // at 1024, 5.54 : 5.43 at 1500, 5.84 : 5.69 at 2048, 6.71 : 6.46 at 3000, 7.41 : 6.93 at 4096; 64 Q / 8 KV heads
            // (8 wavefronts) 5.09 : 5.22 at 512, 5.55 : 5.51 at 1024, 6.35 : 6.13 at 2048, 7.63 : 7.43 at 4096, 10.45 : 9.67 at
            // 8192, 16.07 : 14.72 at 16384.
            const int full = half * 4 + 1;
            want = tiles >= full ? target : tiles >= half ? half : quarter;
            if (want > tiles) want = tiles;
            if (cap < 2) return LLMI_ERR_WORKSPACE;
            if ((size_t)want > cap) want = (int)cap;
        }
        // The kernel deals the tiles to the splits in contiguous runs that differ by at most one
        // tile, so no split is empty as long as there are no more splits than tiles.
        num_splits = want < tiles ? want : tiles;
        tiles_per_split = ceil_div(tiles, num_splits);
        if (num_splits > 1) {
            const size_t need = (fused ? per_split_fused : per_split_plain) * (size_t)num_splits + (fused ? 16 : 0);
            if (!a->workspace || a->workspace_bytes < need) return LLMI_ERR_WORKSPACE;
        }
    }
    if (num_splits == 1) {
        path = LLMI_PATH_SINGLE_PASS;
        tiles_per_split = tiles;
        if (a->waves_per_group) {
            waves = a->waves_per_group;
        } else {
            waves = pow2_ceil(tiles);
            if (waves > single_waves_max) waves = single_waves_max;
        }
    }

    p->path = path;
    p->num_splits = num_splits;
    p->rows_per_split = tiles_per_split * kTile;
    p->waves_per_group = waves;
    p->group_pad = group_pad;
    p->workspace_side = 0;
    p->workspace_needed = num_splits <= 1 ? 0
                          : path == LLMI_PATH_SPLIT_FUSED ? per_split_fused * (size_t)num_splits + 16
                                                          : per_split_plain * (size_t)num_splits;
    // The workspace laid out by package side: where every split of a KV head and its combiner run on one XCD (the KV
    // head is the fastest grid index and the head count a multiple of the eight XCDs), where one wavefront merges
    // a head (the shared read-back of larger groups keeps the plain layout), with the wave count the dispatcher picks
    // itself (the only ones the kernel is built for in this layout), and where the workspace has room
    // for two homes per row, rounded to whole 8 KiB blocks, behind the way to the next 16 KiB boundary. Otherwise the
    // plain layout, silently: the side only ever changes the time.
    if (path == LLMI_PATH_SPLIT_FUSED && num_splits > 1 && a->workspace_side != 0 && n_kv % 8 == 0 && a->kv_mul <= waves &&
        a->head_num <= 128 && by_side_variant(group_pad, waves)) {
        const size_t need = side_pad(a->workspace) + fused_workspace(a->head_num, a->head_dim, num_splits, true).bytes();
        if (a->workspace_bytes >= need) {
            p->workspace_side = 1;
            p->workspace_needed = need;
        }
    }
    return LLMI_OK;
}

}  // namespace llmi

using namespace llmi;

extern "C" {

int llmi_hip_mha_plan(const llmi_mha_args* args, llmi_mha_plan* plan) {
    if (!plan) return LLMI_ERR_NULL_POINTER;
    return make_plan(args, plan);
}

int llmi_hip_mha_decode(const llmi_mha_args* args) {
    llmi_mha_plan plan;
    if (int rc = make_plan(args, &plan)) return rc;
    return launch_mha_decode(*args, plan);
}

int llmi_hip_mha_decode_static(const llmi_mha_args* args) {
    if (!args) return LLMI_ERR_NULL_POINTER;
    // Plan first, against the size of the static scratch and a stand-in address: an argument or size error
    // comes back before anything touches the device.
    llmi_mha_args a = *args;
    a.workspace = reinterpret_cast<void*>(uintptr_t{256});
    a.workspace_bytes = LLMI_STATIC_SCRATCH_BYTES;
    llmi_mha_plan plan;
    if (int rc = make_plan(&a, &plan)) {
        if (rc == LLMI_ERR_WORKSPACE)
            g_last_error = "llmi_hip_mha_decode_static: this head count / split count needs more than the " +
                           std::to_string(LLMI_STATIC_SCRATCH_BYTES) + "-byte static workspace; use llmi_hip_mha_decode";
        return rc;
    }
    void* ptr = nullptr;
    size_t bytes = 0;
    if (int rc = static_scratch(&ptr, &bytes)) return rc;
    if (plan.workspace_needed > bytes) return LLMI_ERR_WORKSPACE;  // (make_plan has checked this already)
    a.workspace = ptr;
    a.workspace_bytes = bytes;
    // The array's package side, measured once per device: on the first call that is not being captured.
    {
        constexpr int kMaxDevices = 64;
        static std::atomic<int> measured[kMaxDevices];
        static std::atomic<int32_t> sides_of[kMaxDevices];
        int dev = 0;
        if (int rc = record_hip_error(hipGetDevice(&dev), "hipGetDevice")) return rc;
        int32_t sides = 0;
        if (dev >= 0 && dev < kMaxDevices) {
            if (!measured[dev].load(std::memory_order_acquire)) {
                static std::mutex measuring;  // (two first calls at once would measure through the same lines)
                std::lock_guard<std::mutex> lock(measuring);
                hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
                hipStream_t s = static_cast<hipStream_t>(a.stream);
                if (measured[dev].load(std::memory_order_acquire)) {
                    // (another thread got there first)
                } else if (hipStreamIsCapturing(s, &cs) == hipSuccess && cs == hipStreamCaptureStatusNone) {
                    int32_t found = 0;
                    if (int rc = measure_workspace_side(ptr, bytes, s, &found)) return rc;
                    sides_of[dev].store(found, std::memory_order_relaxed);
                    measured[dev].store(1, std::memory_order_release);
                } else {
                    (void)hipGetLastError();  // (under capture: this call keeps the plain layout)
                }
            }
            if (measured[dev].load(std::memory_order_acquire)) sides = sides_of[dev].load(std::memory_order_relaxed);
        }
        a.workspace_side = sides;
        if (a.workspace_side != args->workspace_side)
            if (int rc = make_plan(&a, &plan)) return rc;  // (same plan, now with the side's layout if it fits)
    }
    return launch_mha_decode(a, plan);
}

int llmi_hip_mha_decode_append(const llmi_mha_append_args* args) {
    if (!args) return LLMI_ERR_NULL_POINTER;
    if (!args->key_new || !args->value_new || !args->norm_weight || !args->sin_cache || !args->cos_cache)
        return LLMI_ERR_NULL_POINTER;
    const void* ptrs[] = {args->key_new, args->value_new, args->norm_weight, args->sin_cache, args->cos_cache};
    for (const void* p : ptrs)
        if (!aligned16(p)) return LLMI_ERR_ALIGNMENT;
    if (!(args->eps >= 0.0f)) return LLMI_ERR_INVALID_ARG;
    if (args->mha.force_path == LLMI_PATH_SPLIT) return LLMI_ERR_INVALID_ARG;
    llmi_mha_plan plan;
    if (int rc = make_plan(&args->mha, &plan, kMaxWaves, 1)) return rc;
    return launch_mha_decode(args->mha, plan, args);
}

// Compute units of the current device (asked once per process), or 0 if the device cannot be asked.
static int compute_units() {
    static std::atomic<int> cu_count{0};
    int cus = cu_count.load(std::memory_order_relaxed);
    if (cus == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
            (void)hipGetLastError();
            return 0;
        }
        cu_count.store(cus, std::memory_order_relaxed);
    }
    return cus;
}

// Validates the arguments and decides between the one-launch form (*fused = true, plan filled) and the pair.
// Whether the append variant's launch for (m, plan) walks its tiles in step (no staggered walk): the kernels that never
// stagger (one-launch projection, resident multi-layer launch) only take such lengths, so that they give the bits of the
// launches they stand for.
static bool append_walks_in_step(const llmi_mha_args& m, const llmi_mha_plan& plan) {
    const int tiles = (m.pos + kTile - 1) / kTile;  // (the new token's row does not come from the cache)
    const int64_t row_bytes = m.kv_layout == LLMI_KV_LAYOUT_POS_MAJOR ? (int64_t)m.kv_dim * 2 : (int64_t)m.head_dim * 2;
    return stagger_mask(m.kv_layout, (int64_t)(tiles / plan.num_splits) * kTile * row_bytes, tiles % plan.num_splits != 0) == 0;
}

static int plan_oproj(const llmi_attn_oproj_args* args, llmi_mha_plan* plan, bool* fused) {
    if (!args) return LLMI_ERR_NULL_POINTER;
    const llmi_mha_append_args& ap = args->attn;
    if (!ap.key_new || !ap.value_new || !ap.norm_weight || !ap.sin_cache || !ap.cos_cache || !args->o_weight || !args->residual)
        return LLMI_ERR_NULL_POINTER;
    const void* ptrs[] = {ap.key_new, ap.value_new, ap.norm_weight, ap.sin_cache, ap.cos_cache, args->o_weight, args->residual};
    for (const void* p : ptrs)
        if (!aligned16(p)) return LLMI_ERR_ALIGNMENT;
    if (!(ap.eps >= 0.0f) || args->hidden <= 0) return LLMI_ERR_INVALID_ARG;
    if (ap.mha.force_path == LLMI_PATH_SPLIT) return LLMI_ERR_INVALID_ARG;
    if (args->one_launch != 0 && args->one_launch != 1) return LLMI_ERR_INVALID_ARG;
    if (int rc = make_plan(&ap.mha, plan, kMaxWaves, 1)) return rc;
    *fused = false;
    if (!args->one_launch) return LLMI_OK;  // the pair of launches is the default: it is the faster form and waits for nothing
    const llmi_mha_args& m = ap.mha;
    const int n_kv = m.kv_dim / m.head_dim;
    int32_t rows_per_wave = 0, max_k = 0;
    oproj_limits(&rows_per_wave, &max_k);
    const int64_t k = (int64_t)m.head_num * m.head_dim;
    if (m.pos_device || k % 512 != 0 || k > max_k || m.head_num > 128) return LLMI_OK;  // (one wavefront collects the heads' tags, two per lane)
    // every workgroup must be resident at once: the workers wait for the combiners
    const int cus = compute_units();
    if (cus <= 0) return LLMI_OK;
    auto fits = [&](const llmi_mha_plan& p) {
        if (p.path != LLMI_PATH_SPLIT_FUSED || p.num_splits < 2) return false;
        if (p.group_pad > 8 || p.waves_per_group != (p.group_pad == 8 ? 8 : 4)) return false;
        const int64_t worker_waves = (int64_t)n_kv * (p.num_splits - 1) * p.waves_per_group;
        if (args->hidden > rows_per_wave * worker_waves) return false;
        if ((int64_t)n_kv * p.num_splits > cus) return false;
        if (!append_walks_in_step(m, p)) return false;
        return m.workspace_bytes >= p.workspace_needed + (size_t)m.head_num * sizeof(uint32_t);
    };
    if (fits(*plan)) {
        *fused = true;
        return LLMI_OK;
    }
    // The dispatcher's own split count may leave too few idle wavefronts for the rows (it prefers half a grid up to
    // four tiles per wavefront): the one-launch form then asks for one workgroup per CU itself.
    if (m.num_splits == 0 && m.force_path != LLMI_PATH_SINGLE_PASS && plan->num_splits > 1 && cus / n_kv > plan->num_splits) {
        llmi_mha_args wide = m;
        wide.num_splits = cus / n_kv > kMaxSplits ? kMaxSplits : cus / n_kv;
        wide.force_path = LLMI_PATH_SPLIT_FUSED;
        llmi_mha_plan p2;
        if (make_plan(&wide, &p2, kMaxWaves, 1) == LLMI_OK && p2.num_splits == wide.num_splits && fits(p2)) {
            *plan = p2;
            *fused = true;
        }
    }
    return LLMI_OK;
}

int llmi_hip_mha_oproj_launches(const llmi_attn_oproj_args* args) {
    llmi_mha_plan plan;
    bool fused = false;
    if (int rc = plan_oproj(args, &plan, &fused)) return rc;
    return fused ? 1 : 2;
}

int llmi_hip_mha_decode_append_oproj(const llmi_attn_oproj_args* args) {
    llmi_mha_plan plan;
    bool fused = false;
    if (int rc = plan_oproj(args, &plan, &fused)) return rc;
    if (fused) return launch_mha_decode(args->attn.mha, plan, &args->attn, args);
    if (int rc = launch_mha_decode(args->attn.mha, plan, &args->attn)) return rc;
    const llmi_mha_args& m = args->attn.mha;
    void* const out[3] = {args->residual, args->residual, args->residual};
    const int32_t seg_end[3] = {args->hidden, args->hidden, args->hidden};
    return launch_gemv(m.output, args->o_weight, out, seg_end, args->hidden, m.head_num * m.head_dim, LLMI_GEMV_ADD_BF16,
                       static_cast<hipStream_t>(m.stream));
}

// Validates a multi-layer call and decides between the one-launch form (*one_launch = true, plan = layer 0's) and
// one launch per layer.
static int plan_stack(const llmi_mha_stack_args* args, llmi_mha_plan* plan, bool* one_launch) {
    if (!args) return LLMI_ERR_NULL_POINTER;
    const llmi_mha_append_args& ap = args->first;
    if (!ap.key_new || !ap.value_new || !ap.norm_weight || !ap.sin_cache || !ap.cos_cache) return LLMI_ERR_NULL_POINTER;
    const void* ptrs[] = {ap.key_new, ap.value_new, ap.norm_weight, ap.sin_cache, ap.cos_cache};
    for (const void* p : ptrs)
        if (!aligned16(p)) return LLMI_ERR_ALIGNMENT;
    if (!(ap.eps >= 0.0f) || args->layer_count < 1) return LLMI_ERR_INVALID_ARG;
    if (ap.mha.force_path == LLMI_PATH_SPLIT) return LLMI_ERR_INVALID_ARG;
    const int64_t strides[] = {args->query_stride, args->key_new_stride, args->value_new_stride, args->norm_weight_stride,
                               args->output_stride};
    for (int64_t st : strides)
        if (st % 8 != 0) return LLMI_ERR_ALIGNMENT;  // (every layer's rows stay 16-byte aligned)
    if ((int64_t)ap.mha.layer_id + args->layer_count > INT32_MAX) return LLMI_ERR_INVALID_ARG;
    if (int rc = make_plan(&ap.mha, plan, kMaxWaves, 1)) return rc;
    *one_launch = false;
    const llmi_mha_args& m = ap.mha;
    if (m.pos_device) return LLMI_OK;
    if (plan->path != LLMI_PATH_SPLIT_FUSED || plan->num_splits < 2 || plan->num_splits > 64) return LLMI_OK;
    if (plan->group_pad > 4 || plan->waves_per_group != 4 || m.head_num > 64) return LLMI_OK;  // (one lane of the polling wavefront per head)
    if (m.workspace_bytes < plan->workspace_needed + stack_workspace_extra(m.head_num)) return LLMI_OK;
    // every workgroup must be resident at once: workgroups wait for each other
    const int cus = compute_units();
    if (cus <= 0 || (int64_t)(m.kv_dim / m.head_dim) * plan->num_splits > cus) return LLMI_OK;
    // Lengths at which the per-layer launches stagger their walk stay with them: the resident kernel walks in step, so
    // it would neither be as fast there nor give the same bits (the order of a split's tiles is the order of its sums).
    if (!append_walks_in_step(m, *plan)) return LLMI_OK;
    *one_launch = true;
    return LLMI_OK;
}

int llmi_hip_mha_stack_launches(const llmi_mha_stack_args* args) {
    llmi_mha_plan plan;
    bool one = false;
    if (int rc = plan_stack(args, &plan, &one)) return rc;
    return one ? 1 : args->layer_count;
}

int llmi_hip_mha_decode_append_stack(const llmi_mha_stack_args* args) {
    llmi_mha_plan plan;
    bool one = false;
    if (int rc = plan_stack(args, &plan, &one)) return rc;
    if (one) return launch_mha_stack(*args, plan);
    for (int32_t l = 0; l < args->layer_count; ++l) {
        llmi_mha_append_args a = args->first;
        a.mha.layer_id += l;
        a.mha.query = static_cast<const uint16_t*>(a.mha.query) + l * args->query_stride;
        a.key_new = static_cast<const uint16_t*>(a.key_new) + l * args->key_new_stride;
        a.value_new = static_cast<const uint16_t*>(a.value_new) + l * args->value_new_stride;
        a.norm_weight = static_cast<const uint16_t*>(a.norm_weight) + l * args->norm_weight_stride;
        a.mha.output = static_cast<uint16_t*>(a.mha.output) + l * args->output_stride;
        if (a.mha.output_f32) a.mha.output_f32 += l * args->output_stride;
        if (int rc = launch_mha_decode(a.mha, plan, &a)) return rc;
    }
    return LLMI_OK;
}

size_t llmi_hip_mha_workspace_bytes(int32_t head_num, int32_t head_dim, int32_t max_seq_len) {
    if (head_num <= 0 || head_dim <= 0 || max_seq_len <= 0) return 0;
    int splits = (max_seq_len + kTile - 1) / kTile;
    if (splits > kMaxSplits) splits = kMaxSplits;
    // Per head and split: head_dim partial outputs plus either (max, sum) as two floats
    // (separate combine kernel) or two 8-byte arrival records (fused combine).
    // ... and, behind the records, one 4-byte counter per head for the fused output projection.
    // ... and room for the layout by package side: the way to the first 8 KiB boundary, both arrays rounded up to whole
    // blocks per side; never less than what llmi_hip_mha_workspace_side needs for its measurement.
    const size_t plain = (size_t)head_num * (size_t)splits * ((size_t)head_dim * sizeof(float) + 2 * sizeof(unsigned long long)) + 16;
    // (the layout by side exists for the head_dim the kernels take; a row of any other width would not fit its 8 KiB blocks)
    const size_t by_side = head_dim == 128 ? fused_workspace(head_num, head_dim, splits, true).bytes() + 2 * kSideBlock : 0;
    // ... and the multi-layer launch's done tags
    size_t need = (plain > by_side ? plain : by_side) + (size_t)head_num * sizeof(uint32_t) + stack_workspace_extra(head_num);
    if (need < 6 * kSideBlock) need = 6 * kSideBlock;
    return need;
}

int llmi_hip_mha_workspace_side(void* workspace, size_t workspace_bytes, void* stream, int32_t* side) {
    if (!workspace || !side) return LLMI_ERR_NULL_POINTER;
    if (!aligned16(workspace)) return LLMI_ERR_ALIGNMENT;
    if (workspace_bytes < 6 * kSideBlock) return LLMI_ERR_WORKSPACE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (int rc = record_hip_error(hipStreamIsCapturing(s, &cs), "hipStreamIsCapturing")) return rc;
    if (cs != hipStreamCaptureStatusNone) return LLMI_ERR_INVALID_ARG;
    return measure_workspace_side(workspace, workspace_bytes, s, side);
}

int llmi_hip_qk_norm_rope_append(const llmi_qk_norm_rope_args* a) {
    if (!a) return LLMI_ERR_NULL_POINTER;
    if (!a->query || !a->key_new || !a->key_cache || !a->norm_weight || !a->sin_cache || !a->cos_cache)
        return LLMI_ERR_NULL_POINTER;
    if (a->value_new && !a->value_cache) return LLMI_ERR_NULL_POINTER;
    if (a->head_dim != 128) return LLMI_ERR_HEAD_DIM;                                // rmsnorm_kernel.cu:274
    if (a->kv_dim <= 0 || a->kv_dim % a->head_dim != 0) return LLMI_ERR_KV_DIM;
    if (a->head_num <= 0 || a->max_seq_len <= 0 || a->layer_id < 0) return LLMI_ERR_INVALID_ARG;
    if (a->pos < 0 || a->pos >= a->max_seq_len) return LLMI_ERR_POS_RANGE;
    if (a->kv_layout != LLMI_KV_LAYOUT_POS_MAJOR && a->kv_layout != LLMI_KV_LAYOUT_HEAD_MAJOR)
        return LLMI_ERR_LAYOUT;
    const void* ptrs[] = {a->query, a->query_src, a->key_new, a->value_new, a->key_cache, a->value_cache, a->norm_weight};
    for (const void* p : ptrs)
        if (p && (reinterpret_cast<uintptr_t>(p) & 3u)) return LLMI_ERR_ALIGNMENT;
    if (!(a->eps >= 0.0f)) return LLMI_ERR_INVALID_ARG;
    return launch_qk_norm_rope_append(*a);
}

int llmi_hip_sincos_table(float* sin_cache, float* cos_cache, int32_t head_dim, int32_t max_seq_len,
                          void* stream) {
    if (!sin_cache || !cos_cache) return LLMI_ERR_NULL_POINTER;
    if (head_dim <= 0 || head_dim % 2 != 0) return LLMI_ERR_HEAD_DIM;
    if (max_seq_len <= 0) return LLMI_ERR_INVALID_ARG;
    return launch_sincos_table(sin_cache, cos_cache, head_dim, max_seq_len, static_cast<hipStream_t>(stream));
}

int llmi_hip_kv_restride(const void* src, void* dst, int32_t layer_num, int32_t max_seq_len, int32_t kv_dim,
                         int32_t head_dim, int32_t num_pos, void* stream) {
    if (!src || !dst) return LLMI_ERR_NULL_POINTER;
    if (head_dim != 128) return LLMI_ERR_HEAD_DIM;
    if (kv_dim <= 0 || kv_dim % head_dim != 0) return LLMI_ERR_KV_DIM;
    if (layer_num <= 0 || max_seq_len <= 0) return LLMI_ERR_INVALID_ARG;
    if (num_pos < 0 || num_pos > max_seq_len) return LLMI_ERR_POS_RANGE;
    if (!aligned16(src) || !aligned16(dst)) return LLMI_ERR_ALIGNMENT;
    if (src == dst) return LLMI_ERR_INVALID_ARG;
    return launch_kv_restride(src, dst, layer_num, max_seq_len, kv_dim, head_dim, num_pos,
                              static_cast<hipStream_t>(stream));
}

/* ---- pool ---------------------------------------------------------------- */

llmi_pool* llmi_pool_create(llmi_backing_alloc_fn alloc_fn, llmi_backing_free_fn free_fn, void* user) {
    if (!alloc_fn || !free_fn) return nullptr;
    return new (std::nothrow) llmi_pool(alloc_fn, free_fn, user);
}

void llmi_pool_destroy(llmi_pool* pool) { delete pool; }

void* llmi_pool_alloc(llmi_pool* pool, size_t bytes) { return pool ? pool->allocate(bytes) : nullptr; }

int llmi_pool_free(llmi_pool* pool, void* ptr) { return pool ? pool->release(ptr) : LLMI_ERR_NULL_POINTER; }

size_t llmi_pool_trim(llmi_pool* pool) { return pool ? pool->trim() : 0; }

int llmi_pool_get_stats(const llmi_pool* pool, llmi_pool_stats* stats) {
    if (!pool || !stats) return LLMI_ERR_NULL_POINTER;
    pool->stats(stats);
    return LLMI_OK;
}

static int hip_backing_alloc(void** ptr, size_t bytes, void*) {
    hipError_t err = hipMalloc(ptr, bytes);
    if (err != hipSuccess) {
        record_hip_error(err, "hipMalloc");
        (void)hipGetLastError();
        *ptr = nullptr;
        return LLMI_ERR_OUT_OF_MEMORY;
    }
    return 0;
}

static int hip_backing_free(void* ptr, void*) { return record_hip_error(hipFree(ptr), "hipFree"); }

llmi_pool* llmi_hip_default_pool(void) {
    // Leaked on purpose: device memory is reclaimed by the driver at process
    // exit, and freeing from a static destructor can run after HIP has shut down.
    static llmi_pool* pool = new llmi_pool(hip_backing_alloc, hip_backing_free, nullptr);
    return pool;
}

void* llmi_hip_pool_alloc(size_t bytes) { return llmi_hip_default_pool()->allocate(bytes); }

int llmi_hip_pool_free(void* ptr) { return llmi_hip_default_pool()->release(ptr); }

int llmi_hip_memcpy(void* dst, const void* src, size_t bytes, int32_t kind, void* stream, int32_t need_sync) {
    if (!dst || !src) return LLMI_ERR_NULL_POINTER;  // alloc.cpp:12-13
    if (bytes == 0) return LLMI_OK;                  // alloc.cpp:15-17
    if (kind == 0) {
        std::memcpy(dst, src, bytes);  // alloc.cpp:26-27
        return LLMI_OK;
    }
    hipMemcpyKind k;
    if (kind == 1) k = hipMemcpyHostToDevice;
    else if (kind == 2) k = hipMemcpyDeviceToHost;
    else if (kind == 3) k = hipMemcpyDeviceToDevice;
    else return LLMI_ERR_INVALID_ARG;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // A NULL stream copies synchronously, a stream asynchronously (alloc.cpp:28-46).
    hipError_t err = s ? hipMemcpyAsync(dst, src, bytes, k, s) : hipMemcpy(dst, src, bytes, k);
    if (err != hipSuccess) return record_hip_error(err, "hipMemcpy");
    if (need_sync) return record_hip_error(hipDeviceSynchronize(), "hipDeviceSynchronize");
    return LLMI_OK;
}

int llmi_hip_memset_zero(void* ptr, size_t bytes, void* stream, int32_t need_sync) {
    if (!ptr) return LLMI_ERR_NULL_POINTER;
    if (bytes == 0) return LLMI_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t err = s ? hipMemsetAsync(ptr, 0, bytes, s) : hipMemset(ptr, 0, bytes);  // alloc.cpp:61-66
    if (err != hipSuccess) return record_hip_error(err, "hipMemset");
    if (need_sync) return record_hip_error(hipDeviceSynchronize(), "hipDeviceSynchronize");
    return LLMI_OK;
}

int llmi_hip_gemv(const llmi_gemv_args* a) {
    if (!a) return LLMI_ERR_NULL_POINTER;
    if (!a->input || !a->weight || !a->output) return LLMI_ERR_NULL_POINTER;
    if (a->n <= 0 || a->k <= 0 || a->k % 8 != 0) return LLMI_ERR_INVALID_ARG;  // matmul_kernel.cu:128
    if (a->mode != LLMI_GEMV_OUT_BF16 && a->mode != LLMI_GEMV_OUT_F32 && a->mode != LLMI_GEMV_ADD_BF16)
        return LLMI_ERR_INVALID_ARG;
    if (!aligned16(a->input) || !aligned16(a->weight) || !aligned16(a->output)) return LLMI_ERR_ALIGNMENT;  // :123-124
    void* const out[3] = {a->output, a->output, a->output};
    const int32_t seg_end[3] = {a->n, a->n, a->n};
    return launch_gemv(a->input, a->weight, out, seg_end, a->n, a->k, a->mode, static_cast<hipStream_t>(a->stream));
}

int llmi_hip_qkv_gemv(const llmi_qkv_gemv_args* a) {
    if (!a) return LLMI_ERR_NULL_POINTER;
    if (!a->input || !a->weight || !a->query || !a->key || !a->value) return LLMI_ERR_NULL_POINTER;
    if (a->dim <= 0 || a->kv_dim <= 0 || a->k <= 0 || a->k % 8 != 0) return LLMI_ERR_INVALID_ARG;  // :290-292
    if ((int64_t)a->dim + 2 * (int64_t)a->kv_dim > INT32_MAX) return LLMI_ERR_INVALID_ARG;
    const void* ptrs[] = {a->input, a->weight, a->query, a->key, a->value};
    for (const void* p : ptrs)
        if (!aligned16(p)) return LLMI_ERR_ALIGNMENT;
    void* const out[3] = {a->query, a->key, a->value};
    const int32_t seg_end[3] = {a->dim, a->dim + a->kv_dim, a->dim + 2 * a->kv_dim};
    return launch_gemv(a->input, a->weight, out, seg_end, seg_end[2], a->k, LLMI_GEMV_OUT_BF16,
                       static_cast<hipStream_t>(a->stream));
}

int llmi_hip_abi_version(void) { return LLMI_HIP_ABI_VERSION; }

int32_t llmi_hip_set_test_far_home(int32_t mode) {
    return llmi::g_test_far_home.exchange(mode < 0 || mode > 2 ? 0 : mode, std::memory_order_relaxed);
}

int32_t llmi_hip_stagger_mask(int32_t kv_layout, int64_t run_bytes, int32_t ragged) {
    return llmi::stagger_mask(kv_layout, run_bytes, ragged != 0);
}

int32_t llmi_hip_set_poll_limit(int32_t polls) {
    return llmi::g_poll_limit.exchange(polls < 0 ? 0 : polls, std::memory_order_relaxed);
}

int llmi_hip_poll_timeouts(uint64_t* count) {
    if (!count) return LLMI_ERR_NULL_POINTER;
    unsigned long long n = 0;
    if (int rc = read_poll_timeouts(&n)) return rc;
    *count = n;
    return LLMI_OK;
}

const char* llmi_hip_strerror(int status) {
    switch (status) {
        case LLMI_OK: return "ok";
        case LLMI_ERR_NULL_POINTER: return "required pointer is NULL";
        case LLMI_ERR_HEAD_DIM: return "head_dim must be 128";
        case LLMI_ERR_KV_DIM: return "kv_dim must be a positive multiple of head_dim";
        case LLMI_ERR_ALIGNMENT: return "pointer is not sufficiently aligned (16 bytes for q/K/V/out/workspace)";
        case LLMI_ERR_POS_RANGE: return "pos out of range [0, max_seq_len)";
        case LLMI_ERR_WORKSPACE: return "split workspace missing or too small";
        case LLMI_ERR_HEAD_GROUP: return "head_num must equal kv_mul * kv_heads with 1 <= kv_mul <= 16";
        case LLMI_ERR_LAYOUT: return "unknown kv_layout";
        case LLMI_ERR_INVALID_ARG: return "argument out of range";
        case LLMI_ERR_LAUNCH: return "HIP call or kernel launch failed (see llmi_hip_last_error)";
        case LLMI_ERR_UNKNOWN_POINTER: return "pointer is not a busy block of this pool";
        case LLMI_ERR_OUT_OF_MEMORY: return "backing allocator failed";
        default: return "unknown status";
    }
}

const char* llmi_hip_last_error(void) { return g_last_error.c_str(); }

}  // extern "C"
