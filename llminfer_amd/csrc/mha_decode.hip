// Decode-phase grouped-query attention for gfx950 (MI355X), batch 1: the host side of the kernels of
// mha_decode_kernels.h -- argument block, choice of the instantiation, the static split workspace -- and the
// separate log-sum-exp combine kernel. The kernels themselves are instantiated per query-group size in
// mha_decode_group*.hip.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "llmi_internal.h"
#include "mha_decode_args.h"
#include "wave_ops.h"

// Split workspace of llmi_hip_mha_decode_static, for callers that cannot allocate: part of the code
// object, so every GPU the library runs on holds its own copy from the moment the code object is loaded
// there until the process ends. In host code the name below only stands for the symbol; the
// device address comes from hipGetSymbolAddress (static_scratch() below), once per device.
static __device__ __align__(256) unsigned char scratch[LLMI_STATIC_SCRATCH_BYTES];
namespace llmi {

namespace {

constexpr int kTile = 16;      // positions per MFMA tile
constexpr int kHeadDim = 128;
// Fused output projection: weight rows a wavefront holds in registers while it waits for the attention
// output, and 512-element steps per row (kOprojSteps * 512 = the widest attention output it takes).
// (the same constants as in mha_decode_kernels.h)
constexpr int kOprojRows = 3;
constexpr int kOprojSteps = 8;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
// Round to nearest even, NaN kept quiet.
__device__ __forceinline__ uint16_t f32_to_bf16(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    if (x != x) return 0x7fc0;
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// Log-sum-exp merge of the split partials of one query head
// (role of flashdecoding_gqa_combine_kernel, mha_kernel.cu:399-438).
__global__ __launch_bounds__(kHeadDim) void mha_combine_kernel(const float* __restrict__ ws,
                                                                uint16_t* __restrict__ out,
                                                                float* __restrict__ out_f32, int32_t n_q,
                                                                int32_t num_splits) {
    __shared__ float s_w[kMaxSplits];
    __shared__ float s_red[2];
    const int hq = blockIdx.x;
    const int tid = threadIdx.x;
    const int64_t S = num_splits;
    const float* ms = ws + (int64_t)n_q * S * kHeadDim + (int64_t)hq * S;
    const float* ls = ws + (int64_t)n_q * S * (kHeadDim + 1) + (int64_t)hq * S;

    float mx = -INFINITY;
    for (int s = tid; s < num_splits; s += kHeadDim) mx = fmaxf(mx, ms[s]);
    mx = wave_max(mx);
    if ((tid & 63) == 0) s_red[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(s_red[0], s_red[1]);
    __syncthreads();

    float lsum = 0.0f;
    for (int s = tid; s < num_splits; s += kHeadDim) {
        const float m = ms[s];
        const float f = (m == -INFINITY) ? 0.0f : fast_exp2(m - mx);
        s_w[s] = f;
        lsum += ls[s] * f;
    }
    lsum = wave_sum(lsum);
    if ((tid & 63) == 0) s_red[tid >> 6] = lsum;
    __syncthreads();
    lsum = s_red[0] + s_red[1];

    const float* os = ws + (int64_t)hq * S * kHeadDim + tid;
    float acc = 0.0f;
    for (int s = 0; s < num_splits; ++s) acc += os[(int64_t)s * kHeadDim] * s_w[s];
    const float r = acc / lsum;
    out[(int64_t)hq * kHeadDim + tid] = f32_to_bf16(r);
    if (out_f32) out_f32[(int64_t)hq * kHeadDim + tid] = r;
}
}  // namespace

int oproj_limits(int32_t* rows_per_wave, int32_t* max_k) {
    *rows_per_wave = kOprojRows;
    *max_k = kOprojSteps * 512;
    return LLMI_OK;
}

int static_scratch(void** ptr, size_t* bytes) {
    // One address per device, looked up with that device current the first time it is asked for.
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void* addr[kMaxDevices] = {};
    int dev = 0;
    if (int rc = record_hip_error(hipGetDevice(&dev), "hipGetDevice")) return rc;
    if (dev < 0 || dev >= kMaxDevices) return LLMI_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lock(mu);
    if (!addr[dev]) {
        void* p = nullptr;
        if (int rc = record_hip_error(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return rc;
        if (!p) return LLMI_ERR_LAUNCH;
        addr[dev] = p;
    }
    *ptr = addr[dev];
    *bytes = sizeof(scratch);
    return LLMI_OK;
}

int read_poll_timeouts(unsigned long long* count) {
    // (every translation unit that instantiates the kernels counts on its own device word)
    hipError_t (*const parts[])(unsigned int*) = {poll_timeouts_group1, poll_timeouts_group2, poll_timeouts_group4,
                                                  poll_timeouts_group8, poll_timeouts_group16, poll_timeouts_stack};
    unsigned long long total = 0;
    for (auto part : parts) {
        unsigned int n = 0;
        if (int rc = record_hip_error(part(&n), "hipMemcpyFromSymbol")) return rc;
        total += n;
    }
    *count = total;
    return LLMI_OK;
}

// The kernels' argument block for one call. *fused_end: the first byte behind the fused combine's records in the
// workspace (where the one-launch projection and the multi-layer kernel keep their words), or nullptr.
static int fill_kernel_args(const llmi_mha_args& args, const llmi_mha_plan& plan, const llmi_mha_append_args* append,
                            const llmi_attn_oproj_args* oproj, int tags, KernelArgs* out_ka, char** out_fused_end) {
    const int64_t layer_off = (int64_t)args.layer_id * args.max_seq_len * args.kv_dim;

    KernelArgs ka{};
    ka.q = static_cast<const uint16_t*>(args.query);
    ka.k = static_cast<const uint16_t*>(args.key_cache) + layer_off;
    ka.v = static_cast<const uint16_t*>(args.value_cache) + layer_off;
    ka.ws = static_cast<float*>(args.workspace);
    ka.out = static_cast<uint16_t*>(args.output);
    ka.out_f32 = args.output_f32;
    ka.records = nullptr;
    ka.tag = 0;
    ka.pos_dev = args.pos_device;
    char* fused_end = nullptr;  // behind the records: the fused output projection's words
    if (plan.path == LLMI_PATH_SPLIT_FUSED) {
        // Arrival records sit behind the partial outputs in the workspace; laid out by package side, both arrays
        // start on an 8 KiB boundary.
        const bool by_side = plan.workspace_side != 0 && by_side_variant(plan.group_pad, plan.waves_per_group);
        const FusedWorkspace fw = fused_workspace(args.head_num, args.head_dim, plan.num_splits, by_side);
        char* base = static_cast<char*>(args.workspace);
        if (by_side) {
            const size_t pad = side_pad(args.workspace);
            if (pad + fw.bytes() > args.workspace_bytes) return LLMI_ERR_WORKSPACE;  // (the plan was made for this workspace)
            base += pad;
            ka.by_side = true;
            ka.far_home = test_far_home();
            ka.ws = reinterpret_cast<float*>(base);
            // One rule per head, taken from the region its first row lies in (a head whose rows straddle a region
            // boundary has some of them in far memory, nothing else): two bits per 2 MiB region in workspace_side,
            // counted from the region the workspace starts in, 2 = XCDs 0-3 are nearest to addresses with bit 13 set;
            // a region it says nothing about counts as one of the other kind (any rule does: every workgroup applies the same).
            const uintptr_t region0 = reinterpret_cast<uintptr_t>(args.workspace) >> 21;
            const uint32_t sides = (uint32_t)args.workspace_side;
            auto block_of_side0 = [&](uintptr_t addr) -> unsigned long long {
                const uintptr_t region = (addr >> 21) - region0;
                return region < 16 && ((sides >> (2 * region)) & 3u) == 2u ? 1ull : 0ull;
            };
            const uintptr_t part0 = reinterpret_cast<uintptr_t>(base), rec0 = part0 + fw.partial_bytes;
            for (int h = 0; h < args.head_num && h < 128; ++h) {
                const uintptr_t row = (uintptr_t)h * plan.num_splits;
                ka.ppar[h >> 6] |= block_of_side0(part0 + ((row >> 4) << 14)) << (h & 63);
                ka.rpar[h >> 6] |= block_of_side0(rec0 + ((row >> 9) << 14)) << (h & 63);
            }
        }
        ka.records = reinterpret_cast<unsigned long long*>(base + fw.partial_bytes);
        fused_end = base + fw.partial_bytes + fw.record_bytes;
        // (a multi-layer launch takes one tag per layer, consecutive ones)
        const unsigned long long epoch = next_epoch();
        for (int i = 1; i < tags; ++i) (void)next_epoch();
        ka.tag = record_tag(epoch);
    }
    if (args.kv_layout == LLMI_KV_LAYOUT_POS_MAJOR) {
        ka.row_stride = args.kv_dim;
        ka.head_stride = args.head_dim;
    } else {
        ka.row_stride = args.head_dim;
        ka.head_stride = (int64_t)args.max_seq_len * args.head_dim;
    }
    ka.seq_len = args.pos + 1;
    ka.spread_merge = plan.num_splits >= spread_merge_min_splits(plan.group_pad);
    ka.max_polls = poll_limit();
    ka.stagger = 0;  // (decided below, once the runs of the splits are known)
    ka.group = args.kv_mul;
    ka.n_q = args.head_num;
    ka.num_splits = plan.num_splits;
    {
        const int cached = args.pos + 1 - (append ? 1 : 0);
        const int tiles = (cached + kTile - 1) / kTile;
        ka.tiles_run = tiles / plan.num_splits;
        ka.tiles_longer = tiles % plan.num_splits;
        // (where the splits' runs start a multiple of 512 KiB apart the splits start their walks at different tiles)
        const int64_t run_bytes = (int64_t)ka.tiles_run * kTile * ka.row_stride * 2;
        ka.stagger = args.pos_device ? dyn_stagger(args.kv_layout, run_bytes)  // (pos is the upper bound here)
                                     : stagger_mask(args.kv_layout, run_bytes, ka.tiles_longer != 0);
    }
    ka.scale_log2e = 1.4426950408889634f / sqrtf((float)args.head_dim);
    if (append) {
        ka.k_new = static_cast<const uint16_t*>(append->key_new);
        ka.v_new = static_cast<const uint16_t*>(append->value_new);
        ka.norm_w = static_cast<const uint16_t*>(append->norm_weight);
        ka.sin_cache = append->sin_cache;
        ka.cos_cache = append->cos_cache;
        ka.slot_head_stride = ka.head_stride;
        ka.eps = append->eps;
    }
    if (oproj) {
        // The generation word and the per-head tags sit behind the arrival records (the caller has checked that they fit).
        ka.ready = reinterpret_cast<uint32_t*>(fused_end);
        ka.o_w = static_cast<const uint16_t*>(oproj->o_weight);
        ka.o_res = static_cast<uint16_t*>(oproj->residual);
        ka.o_n = oproj->hidden;
    }
    *out_ka = ka;
    if (out_fused_end) *out_fused_end = fused_end;
    return LLMI_OK;
}

size_t stack_workspace_extra(int head_num) { return 256 + stack_done_bytes(head_num); }

int launch_mha_stack(const llmi_mha_stack_args& st, const llmi_mha_plan& plan) {
    const llmi_mha_args& m = st.first.mha;
    StackArgs sa{};
    char* fused_end = nullptr;
    if (int rc = fill_kernel_args(m, plan, &st.first, nullptr, st.layer_count, &sa.a, &fused_end)) return rc;
    if (!fused_end) return LLMI_ERR_INVALID_ARG;  // (the caller has checked: fused split path)
    sa.layers = st.layer_count;
    sa.q_stride = st.query_stride;
    sa.knew_stride = st.key_new_stride;
    sa.vnew_stride = st.value_new_stride;
    sa.normw_stride = st.norm_weight_stride;
    sa.out_stride = st.output_stride;
    sa.cache_stride = (int64_t)m.max_seq_len * m.kv_dim;
    // the heads' done tags: behind the records, on a 256-byte line of their own
    sa.done = reinterpret_cast<uint32_t*>((reinterpret_cast<uintptr_t>(fused_end) + 255u) & ~(uintptr_t)255u);
    if (!launch_stack(sa, m.kv_dim / m.head_dim, plan.group_pad, plan.waves_per_group, static_cast<hipStream_t>(m.stream)))
        return LLMI_ERR_INVALID_ARG;
    return check_launch();
}

int launch_mha_decode(const llmi_mha_args& args, const llmi_mha_plan& plan, const llmi_mha_append_args* append,
                      const llmi_attn_oproj_args* oproj) {
    const int n_kv = args.kv_dim / args.head_dim;
    KernelArgs ka{};
    if (int rc = fill_kernel_args(args, plan, append, oproj, 1, &ka, nullptr)) return rc;

    hipStream_t stream = static_cast<hipStream_t>(args.stream);
    const bool ap = append != nullptr;
    bool ok = false;
    if (oproj) {
        // (the caller has checked the shape: fused split path, 4 waves, or 8 for groups of 8 heads)
        switch (plan.group_pad) {
            case 1: ok = launch_oproj_group1(ka, n_kv, plan.waves_per_group, stream); break;
            case 2: ok = launch_oproj_group2(ka, n_kv, plan.waves_per_group, stream); break;
            case 4: ok = launch_oproj_group4(ka, n_kv, plan.waves_per_group, stream); break;
            case 8: ok = launch_oproj_group8(ka, n_kv, plan.waves_per_group, stream); break;
            default: ok = false;
        }
        if (!ok) return LLMI_ERR_INVALID_ARG;
        return check_launch();
    }
    switch (plan.group_pad) {
        case 1: ok = launch_decode_group1(ka, n_kv, plan.waves_per_group, ap, stream); break;
        case 2: ok = launch_decode_group2(ka, n_kv, plan.waves_per_group, ap, stream); break;
        case 4: ok = launch_decode_group4(ka, n_kv, plan.waves_per_group, ap, stream); break;
        case 8: ok = launch_decode_group8(ka, n_kv, plan.waves_per_group, ap, stream); break;
        case 16: ok = launch_decode_group16(ka, n_kv, plan.waves_per_group, ap, stream); break;
        default: ok = false;
    }
    if (!ok) return LLMI_ERR_INVALID_ARG;
    if (int rc = check_launch()) return rc;

    if (plan.num_splits > 1 && plan.path != LLMI_PATH_SPLIT_FUSED) {
        hipLaunchKernelGGL(mha_combine_kernel, dim3(args.head_num), dim3(kHeadDim), 0, stream, ka.ws, ka.out,
                           ka.out_f32, args.head_num, plan.num_splits);
        if (int rc = check_launch()) return rc;
    }
    return LLMI_OK;
}

}  // namespace llmi
