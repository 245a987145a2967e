// The attention of SEVERAL consecutive layers of one decode step in ONE launch, for gfx950 (MI355X):
// per layer the fused QK-Norm + RoPE, the K/V append and grouped-query attention over positions 0..pos --
// what the layer loop of the reference issues as one pair of kernels per layer
// (code/source/model/qwen3_fused.cpp:115-127 with :524-548; kernels rmsnorm_kernel.cu:205-290 and
// mha_kernel.cu:440-529), and what llmi_hip_mha_decode_append does per layer here.
//
// Why one launch: at 4096 positions a layer's K and V (16 MiB) stream in about 3 us, but a launch spends 2-3 us
// before its first byte arrives and as long again between its last byte and its result, with HBM idle. Here the
// grid stays resident and walks the layers itself:
//   * the grid is the split path's, one workgroup per (KV head, split) and at most one per compute unit; a wavefront
//     streams its tiles through its ring of LDS slots as one continuous sequence over all layers: the moment a tile
//     of layer l has been read out of its slot, the slot is refilled with the wavefront's next tile, which may
//     belong to layer l+1 -- K and V of the next layer do not depend on this layer's result;
//   * what does depend on it waits for it: layer l+1's query, new K row and new V row are loaded -- and its new row
//     is stored to the cache -- only after every query head of layer l has published its "done" tag, which the
//     merging wavefront of a head writes once the head's output is acknowledged by memory. In an engine the query
//     of layer l+1 is computed from the output of layer l; the launch honours that order also when the buffers
//     alias (a layer's query may BE the previous layer's output);
//   * within a layer everything is the split kernel's: online softmax over 16-position tiles on the matrix cores,
//     the merge of a workgroup's wavefronts through LDS, partial results and arrival records handed to the
//     workgroup of the head's last split, which merges them (log-sum-exp) and writes the bf16 output.
// Every wait is bounded (llmi_hip_set_poll_limit): a wait that gives up is counted and poisons the outputs of its
// layer and the following ones with NaN instead of hanging the device; every wavefront reaches the end of the kernel.
// Needs every workgroup of the grid resident at once (the host checks the grid against the compute unit count).

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mha_device_helpers.h"

namespace llmi {
namespace {

#ifndef LLMI_STACK_PREFETCH_LATE
// 0: a ring slot is refilled with the wavefront's next tile (of the next layer, at the end of a layer) as soon as it
//    has been read; 1: tiles of the NEXT layer are requested only after the wavefront has handed this layer's
//    partial results over.
#define LLMI_STACK_PREFETCH_LATE 0
#endif

#ifndef LLMI_STACK_SPREAD_MERGE
#define LLMI_STACK_SPREAD_MERGE 1  // the heads of a KV head are merged by different workgroups (see `spread` below)
#endif
#ifndef LLMI_STACK_TIMING_NO_WAIT
// 1: timing-only build that does not wait for the previous layer's tags (wrong whenever a layer's inputs depend on the
// layer before): what the order between layers costs. Never the library's build.
#define LLMI_STACK_TIMING_NO_WAIT 0
#endif

#ifndef LLMI_STACK_STAMPS
// 1: diagnostic build that writes the 100 MHz clock at the phases of four layers (LLMI_STACK_STAMP_LAYER ..+3) into the
// caller's workspace, 4 MiB in (the workspace must be at least 4 MiB + 64 KiB + 16 * grid bytes): per layer and
// workgroup 16 words -- 0 tags seen, 1 operands landed, 2 tiles done, 3 partial results handed over, 4 records in,
// 5 partial rows read back, 6 output acknowledged and tag published (4-6: head 0 of a merging workgroup), 8..11 tiles
// done per wavefront. Never the library's build.
#define LLMI_STACK_STAMPS 0
#endif
#ifndef LLMI_STACK_STAMP_LAYER
#define LLMI_STACK_STAMP_LAYER 16
#endif
#if LLMI_STACK_STAMPS
#define LLMI_STAMP(slot, cond)                                                                                          \
    do {                                                                                                                 \
        const int stamp_l_ = layer - LLMI_STACK_STAMP_LAYER;                                                             \
        if (stamp_l_ >= 0 && stamp_l_ < 4 && lane == 0 && (cond)) {                                                      \
            const int stamp_wg_ = (int)blockIdx.y * (int)gridDim.x + (int)blockIdx.x;                                    \
            const int stamp_i_ = ((stamp_l_ * (int)(gridDim.x * gridDim.y) + stamp_wg_) * 16 + (slot)) & ((1 << 18) - 1); \
            reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(a.ws) + (4u << 20))[stamp_i_] = (uint32_t)wall_clock64();   \
        }                                                                                                                \
    } while (0)
#else
#define LLMI_STAMP(slot, cond) do {} while (0)
#endif

// Copies of a head's done tag, each in a 256-byte line of its own: a workgroup polls copy
// (its index in the grid) % kDoneCopies, so that a line is polled by a few workgroups instead of all of them.
#ifndef LLMI_STACK_DONE_COPIES
#define LLMI_STACK_DONE_COPIES 16
#endif
constexpr int kDoneCopies = LLMI_STACK_DONE_COPIES;
static_assert(kDoneCopies >= 1 && kDoneCopies <= 64, "one lane of the merging wavefront writes each copy");
constexpr int kDoneLineWords = 64;  // 256 bytes: room for 64 heads' tags per copy (128 heads: two lines per copy)

template <int G, int NW, int NSTAGE, bool BYSIDE>
__global__ __launch_bounds__(NW * 64, 2) void mha_stack_kernel(StackArgs sa) {
    const KernelArgs& a = sa.a;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n16 = lane & 15;  // MFMA column / DPP-row lane
    const int kg = lane >> 4;   // MFMA k-group / DPP row
    const int kvh = blockIdx.x;  // (the KV head is the fastest grid index: a head's splits and its merging workgroup share an XCD)
    const int split = blockIdx.y;
    const int S = a.num_splits;  // every split holds positions: the host asks for no more splits than tiles

    // The same positions in every layer: tiles 0 .. pos-1 come from the cache, the new token's row from registers.
    const int seq_len = a.seq_len;
    const int cached_len = seq_len - 1;
    const int run = a.tiles_run, longer = a.tiles_longer;  // splits 0 .. longer-1 take run + 1 tiles
    const int ntiles = run + (split < longer ? 1 : 0);
    const int begin = (split * run + min(split, longer)) * kTile;
    const int nrows = min(ntiles * kTile, cached_len - begin);
    // Who merges a query head's splits (log-sum-exp): with at least as many splits as heads in the group, head h's are
    // merged by wavefront 0 of the workgroup of split S-1-h, so that the heads' read-backs run on different compute
    // units at the same time; else the workgroup of the last split merges every head, a wavefront each.
    const bool spread = LLMI_STACK_SPREAD_MERGE && S >= a.group;
    const int merge_head = spread ? (S - 1 - split < a.group ? S - 1 - split : -1) : -1;
    const bool merges_any = spread ? merge_head >= 0 : split == S - 1;
    const bool holds_new_row = split == S - 1 && wave == 0;  // this wavefront takes the new token

    const int64_t split_off = (int64_t)kvh * a.head_stride + (int64_t)begin * a.row_stride;
    const uint32_t rs = (uint32_t)a.row_stride * 2u;
    const uint32_t last_off = (uint32_t)(nrows - 1) * rs;
    const uint32_t k_row = (uint32_t)kg * rs;
    const uint32_t k_col0 = (uint32_t)(n16 ^ kg) * 16u;
    const uint32_t k_col1 = (uint32_t)(n16 ^ (4 + kg)) * 16u;
    const uint32_t k_rd = (uint32_t)((n16 >> 2) * 1024 + (n16 & 3) * 256);
    const uint32_t k_rd0 = k_rd + (uint32_t)((kg ^ (n16 & 7)) * 16);
    const uint32_t k_rd1 = k_rd + (uint32_t)(((4 + kg) ^ (n16 & 7)) * 16);
    const uint32_t v_col = (uint32_t)n16 * 16u;

    // LDS: the wavefronts' rings; the staging of a layer's small operands (norm weights, sin / cos row, new K and V
    // row, the wavefronts' query rows: 1 KiB slots filled by DMA); the wavefronts' partial outputs for the merge; the
    // per-wavefront and merged (max, sum) pairs, the weights of the log-sum-exp merge and the flag of the wait.
    // Just under 80 KiB for groups of four heads: above that the compiler assumes one wavefront per SIMD and moves the
    // accumulators of the matrix products into AGPRs.
    constexpr int kStageBytes = 8192;
    constexpr int kWaveRingBytes = NSTAGE * kStageBytes;
    constexpr int kRingBytes = NW * kWaveRingBytes;
    constexpr int kQSlots = (G * 16 + 63) / 64;
    constexpr int kStagingBytes = (2 + NW * kQSlots) * 1024;
    constexpr int kMergeBytes = NW * G * kHeadDim * (int)sizeof(float);
    constexpr int kTailFloats = 2 * NW * G + 2 * G + G * 64 + 4;
    constexpr int kSmemBytes = kRingBytes + kStagingBytes + kMergeBytes + kTailFloats * 4;
    static_assert(NW > 4 || kSmemBytes <= 80 * 1024, "two workgroups' worth of LDS per CU keeps the VGPR-form matrix instructions");
    static_assert(kSmemBytes <= 160 * 1024, "LDS of one compute unit");
    __shared__ __attribute__((aligned(1024))) char smem[kSmemBytes];
    char* my_ring = smem + wave * kWaveRingBytes;
    const uint32_t my_ring_lds = (uint32_t)(uintptr_t)my_ring;
    char* shared_staging = smem + kRingBytes;
    char* my_rows = shared_staging + (2 + wave * kQSlots) * 1024;
    char* merge_area = smem + kRingBytes + kStagingBytes;
    typedef float (*MergeS)[G];
    auto s_o = [&](int w, int h) { return reinterpret_cast<float*>(merge_area) + (w * G + h) * kHeadDim; };
    MergeS s_m = reinterpret_cast<MergeS>(merge_area + kMergeBytes);
    MergeS s_l = s_m + NW;
    float* s_fin = reinterpret_cast<float*>(s_l + NW);   // [G][2]: merged (max, sum) per head
    float* s_w = s_fin + 2 * G;                          // [G][64] weights of the merge
    int* s_flag = reinterpret_cast<int*>(s_w + G * 64);  // [0]: the previous layer's tags were all seen

    // ---- the stream: this wavefront's tiles of all layers, one sequence ----
    const int n_my = wave < ntiles ? (ntiles - wave + NW - 1) / NW : 0;  // tiles per layer
    int iss_layer = 0, iss_i = 0;  // the next tile to request: tile wave + iss_i * NW of layer iss_layer
    int in_flight = 0;             // tiles requested and not yet read out of their slot
    int iss_stage = 0;
    auto issue_next = [&]() {
        if (n_my == 0 || iss_layer >= sa.layers) return;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the slot's previous contents have reached the VGPRs
        const char* kb = reinterpret_cast<const char*>(a.k + (int64_t)iss_layer * sa.cache_stride + split_off);
        const char* vb = reinterpret_cast<const char*>(a.v + (int64_t)iss_layer * sa.cache_stride + split_off);
        const uint32_t base = (uint32_t)(wave + iss_i * NW) * (kTile * rs);
        const uint32_t slot = my_ring_lds + (uint32_t)iss_stage * kStageBytes;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t ko = min(base + k_row + (uint32_t)(4 * i) * rs, last_off) + ((i & 1) ? k_col1 : k_col0);
            dma16(kb, ko, slot + i * 1024);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t vo = min(base + k_row + (uint32_t)(4 * i) * rs, last_off) + v_col;
            dma16(vb, vo, slot + 4096 + i * 1024);
        }
        ++in_flight;
        iss_stage = (iss_stage + 1 == NSTAGE) ? 0 : iss_stage + 1;
        if (++iss_i == n_my) {
            iss_i = 0;
            ++iss_layer;
        }
    };
    // (a request may belong to the next layer: see LLMI_STACK_PREFETCH_LATE)
    auto issue_within = [&](int layer) {
        if (!LLMI_STACK_PREFETCH_LATE || iss_layer <= layer) issue_next();
    };

    auto read_tile = [&](int stage, TileRegs& r) {
        const char* kp = my_ring + stage * kStageBytes;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            r.k[j] = *reinterpret_cast<const u32x4*>(kp + ((j & 1) ? k_rd1 : k_rd0) + (j >> 1) * 128);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            r.v[i] = *reinterpret_cast<const u32x4*>(kp + 4096 + kg * 1024 + i * 256 + n16 * 16);
    };

    // Where this split's partial results and records go (the same rows in every layer: a layer's are consumed
    // before the next layer's are written, and a record names its layer by its tag).
    const int my_xs = package_side<BYSIDE>();
    const int store_xs = my_xs ^ (int)(BYSIDE && !merges_any && (a.far_home == 1 || (a.far_home == 2 && (split & 1))));
    const int64_t part_rows = BYSIDE ? 2 * (((int64_t)a.n_q * S + 15) & ~(int64_t)15) : (int64_t)a.n_q * S;
    const int part_bytes = (int)(part_rows * kHeadDim * (int64_t)sizeof(float));
    const __amdgpu_buffer_rsrc_t part_rsrc = __builtin_amdgcn_make_buffer_rsrc(a.ws, 0, part_bytes, 0x00020000);
    const int n_units = a.group * (kHeadDim / 4);
    // (NW * 64 threads cover G * 32 units: one unit per thread at most, since G <= NW)
    const int u_h = (int)threadIdx.x >> 5, u_c4 = (int)threadIdx.x & 31;
    const int u_hq = kvh * a.group + min(u_h, a.group - 1);
    const WsHead u_wh = ws_head<BYSIDE>(a, u_hq);
    const uint32_t u_po = (uint32_t)(((int64_t)ws_row<4>(u_wh, split, store_xs) * kHeadDim + u_c4 * 4) * (int64_t)sizeof(float));
    const int64_t u_rec = (int64_t)ws_row<9>(u_wh, split, store_xs) * 2;
    const bool u_own = spread ? merge_head == u_h : split == S - 1;  // this workgroup merges the unit's head itself

    // The done tags: copy c of head h at done[c * words_per_copy + h].
    const int words_per_copy = ((a.n_q + kDoneLineWords - 1) / kDoneLineWords) * kDoneLineWords;
    const uint32_t* my_done = sa.done + (size_t)(((int)blockIdx.y * (int)gridDim.x + (int)blockIdx.x) % kDoneCopies) * words_per_copy;

    int rd_stage = 0;       // the slot the wavefront's next tile is in
    bool poisoned = false;  // a wait gave up: this workgroup's results of this layer and the following are NaN
    for (int s0 = 0; s0 < NSTAGE; ++s0) issue_next();

    for (int layer = 0; layer < sa.layers; ++layer) {
        const uint32_t tag = 0x80000000u | ((a.tag + (uint32_t)layer) & 0x7fffffffu);
        // ---- (1) the previous layer is done: every query head carries its tag ----
        if (!LLMI_STACK_TIMING_NO_WAIT && layer > 0 && wave == 0 && !poisoned) {  // (after a give-up nothing is waited for any more: the rest is NaN anyway)
            const uint32_t want = 0x80000000u | ((a.tag + (uint32_t)layer - 1u) & 0x7fffffffu);
            bool seen = false;
            // (one poll at a time, back to back: two, four or eight polls in flight a fraction of a round trip apart see a
            // tag sooner on paper, and measured 0.06, 0.17 and 0.34 us per layer SLOWER -- polls are traffic on the lines
            // the tags have to reach)
            const uint32_t* tag_ptr = my_done + min(lane, a.n_q - 1);
            for (int spin = 0; spin < a.max_polls && !seen; ++spin)
                seen = __all(__hip_atomic_load(tag_ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == want);
            if (lane == 0) {
                *s_flag = seen ? 1 : 0;
                if (!seen) atomicAdd(&g_poll_timeouts, 1u);
            }
        }
        // (also: every wavefront is through with the previous layer's merge area and staging slots)
        __syncthreads();
        if (!LLMI_STACK_TIMING_NO_WAIT && layer > 0 && *s_flag == 0) poisoned = true;
        LLMI_STAMP(0, wave == 0);

        // ---- (2) this layer's small operands, by DMA into the staging slots ----
        const uint16_t* q_l = a.q + (int64_t)layer * sa.q_stride;
        const int c16 = lane & 15, which = lane >> 4;
        {
            const uint32_t st = (uint32_t)(uintptr_t)shared_staging;
            const uint32_t st_rows = (uint32_t)(uintptr_t)my_rows;
            const float* sin_row = a.sin_cache + (int64_t)(seq_len - 1) * 64;
            const float* cos_row = a.cos_cache + (int64_t)(seq_len - 1) * 64;
            const uint64_t w_base = reinterpret_cast<uint64_t>(a.norm_w + (int64_t)layer * sa.normw_stride) + (uint64_t)(which & 1) * 256u;
            const uint64_t t_base = reinterpret_cast<uint64_t>(which == 2 ? sin_row : cos_row);
            const uint64_t p0 = (which < 2 ? w_base : t_base) + (uint64_t)c16 * 16u;
            dma16_gather(reinterpret_cast<const void*>(p0), st);
            if (holds_new_row) {
                const uint16_t* kn = a.k_new + (int64_t)layer * sa.knew_stride;
                const uint16_t* vn = a.v_new + (int64_t)layer * sa.vnew_stride;
                const uint64_t p1 = reinterpret_cast<uint64_t>((which & 1) == 0 ? kn : vn) + (uint64_t)(kvh * kHeadDim * 2 + c16 * 16);
                dma16_gather_coherent(reinterpret_cast<const void*>(p1), st + 1024);
            }
#pragma unroll
            for (int i = 0; i < kQSlots; ++i) {
                const int head = min(which + 4 * i, a.group - 1);
                dma16_gather_coherent(q_l + (int64_t)(kvh * a.group + head) * kHeadDim + c16 * 8, st_rows + i * 1024);
            }
        }
        // (loads complete in order: the tiles requested earlier are in their slots as well)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        u32x4 qb[4];
        u32x4 new_k[4], new_v;  // the new token's K row (operand layout) and V row, in the wavefront that holds it
        LLMI_STAMP(1, wave == 0);
        float m_run = -INFINITY, l_run = 0.0f;
        f32x4 o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        {
            const u32x4* sh4 = reinterpret_cast<const u32x4*>(shared_staging);
            const u32x4* rows4 = reinterpret_cast<const u32x4*>(my_rows);
#pragma unroll
            for (int b4 = 0; b4 < kQSlots; ++b4)
                norm_rope_rows_lds(my_rows, shared_staging, shared_staging + 512, shared_staging + 768, 4 * b4 + kg, n16, a.eps);
            if (holds_new_row)
                norm_rope_rows_lds(shared_staging + 1024, shared_staging + 256, shared_staging + 512, shared_staging + 768, 0, n16, a.eps);
            const int hq_local = min(n16, a.group - 1);
            const bool live = n16 < a.group;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const u32x4 qv = rows4[hq_local * 16 + j * 4 + kg];
                qb[j] = live ? qv : u32x4{0u, 0u, 0u, 0u};
            }
            if (holds_new_row) {
                // The new token: its K row (normalised + rotated above) and V row go to the cache slot of this layer, and
                // the running softmax starts from that one position -- score q.k, weight 1, output = the V row.
                typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
                u32x4 kf[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) kf[j] = sh4[64 + j * 4 + kg];
                const u32x4 vf = sh4[64 + 16 + n16];
#pragma unroll
                for (int j = 0; j < 4; ++j) new_k[j] = kf[j];
                new_v = vf;  // (filed in the cache behind the tiles: the stores' acknowledgement must not sit in front of a tile's wait)
                float dot = 0.0f;
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const uint32_t qw = qb[j][c], kw = kf[j][c];
                        dot = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, qw), __builtin_bit_cast(bf16x2, kw), dot, false);
                    }
                dot = rows_sum(dot);
                m_run = dot * a.scale_log2e;
                l_run = kg == 0 ? 1.0f : 0.0f;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t vw = vf[j >> 1];
                    const float vj = (j & 1) ? bf16_hi(vw) : bf16_lo(vw);
                    o[j] = f32x4{vj, vj, vj, vj};
                }
            }
        }

        // ---- (3) this layer's tiles ----
        for (int i = 0; i < n_my; ++i) {
            TileRegs r;
            // tile i of this layer is the oldest request in flight: in_flight - 1 newer ones may still be travelling
            wait_tiles_in_flight(in_flight - 1);
            read_tile(rd_stage, r);
            rd_stage = (rd_stage + 1 == NSTAGE) ? 0 : rd_stage + 1;
            --in_flight;
            issue_within(layer);
            // q.K^T, online softmax, P^T.V on the matrix cores (the probabilities as hi + lo bf16)
            f32x4 c = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int j = 0; j < 4; ++j)
                c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, r.k[j]), __builtin_bit_cast(bf16x8, qb[j]), c, 0, 0, 0);
            const int row0 = (wave + i * NW) * kTile + 4 * kg;
            float s[4];
            float tmax = -INFINITY;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                s[e] = (row0 + e < nrows) ? c[e] * a.scale_log2e : -INFINITY;
                tmax = fmaxf(tmax, s[e]);
            }
            tmax = rows_max(tmax);
            const float m_new = fmaxf(m_run, tmax);
            const float alpha = fast_exp2(m_run - m_new);
            float p[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) p[e] = fast_exp2(s[e] - m_new);
            l_run = l_run * alpha + ((p[0] + p[1]) + (p[2] + p[3]));
            m_run = m_new;
            const uint32_t p01 = pack_bf16(p[0], p[1]);
            const uint32_t p23 = pack_bf16(p[2], p[3]);
            const uint32_t q01 = pack_bf16(p[0] - bf16_lo(p01), p[1] - bf16_hi(p01));
            const uint32_t q23 = pack_bf16(p[2] - bf16_lo(p23), p[3] - bf16_hi(p23));
            if (__any(alpha != 1.0f)) {
                static_for<0, 4>([&](auto rr) {
                    const float ar = row_bcast<rr.value>(alpha);  // (G <= 4: only DPP row 0 holds heads)
#pragma unroll
                    for (int j = 0; j < 8; ++j) o[j][rr.value] *= ar;
                });
            }
            const i16x4 pa = __builtin_bit_cast(i16x4, u32x2{p01, p23});
            const i16x4 pb = __builtin_bit_cast(i16x4, u32x2{q01, q23});
            i16x4 vb4[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
                const uint32_t b01 = __builtin_amdgcn_perm(r.v[1][j >> 1], r.v[0][j >> 1], sel);
                const uint32_t b23 = __builtin_amdgcn_perm(r.v[3][j >> 1], r.v[2][j >> 1], sel);
                vb4[j] = __builtin_bit_cast(i16x4, u32x2{b01, b23});
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(pa, vb4[j], o[j], 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(pb, vb4[j], o[j], 0, 0, 0);
        }

        if (holds_new_row) {
            const int64_t row_off = (int64_t)layer * sa.cache_stride + (int64_t)(seq_len - 1) * a.row_stride + kvh * a.slot_head_stride;
            if (n16 == 0) {
                uint16_t* kd = const_cast<uint16_t*>(a.k) + row_off;
#pragma unroll
                for (int j = 0; j < 4; ++j) *reinterpret_cast<u32x4*>(kd + (j * 4 + kg) * 8) = new_k[j];
            }
            if (kg == 0) *reinterpret_cast<u32x4*>(const_cast<uint16_t*>(a.v) + row_off + n16 * 8) = new_v;
        }
        LLMI_STAMP(2, wave == 0);
        LLMI_STAMP(8 + wave, true);
        // ---- (4) fold the workgroup's wavefronts, hand the split's partial results over ----
        l_run = rows_sum(l_run);
        if (kg == 0) {
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                if (r4 < G) {
                    float* dst = s_o(wave, r4) + n16 * 8;
                    *reinterpret_cast<f32x4*>(dst) = f32x4{o[0][r4], o[1][r4], o[2][r4], o[3][r4]};
                    *reinterpret_cast<f32x4*>(dst + 4) = f32x4{o[4][r4], o[5][r4], o[6][r4], o[7][r4]};
                }
            }
            if (n16 < G) {
                s_m[wave][n16] = m_run;
                s_l[wave][n16] = l_run;
            }
        }
        __syncthreads();
        if ((int)threadIdx.x < n_units) {
            float mw[NW], lw[NW];
            f32x4 ow[NW];
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                mw[w] = s_m[w][u_h];
                lw[w] = s_l[w][u_h];
                ow[w] = *reinterpret_cast<const f32x4*>(s_o(w, u_h) + u_c4 * 4);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            float mx = -INFINITY;
#pragma unroll
            for (int w = 0; w < NW; ++w) mx = fmaxf(mx, mw[w]);
            f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
            float lsum = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const float f = (mw[w] == -INFINITY) ? 0.0f : fast_exp2(mw[w] - mx);
                acc += ow[w] * f;
                lsum += lw[w] * f;
            }
            if (poisoned) lsum = __builtin_nanf("");
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc), part_rsrc, u_po, 0, kCacheDevice);
            if (!u_own) {
                // the head's record goes out as soon as this wavefront's stores are acknowledged (the 32 columns of a
                // head are stored by one half of one wavefront)
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                if (u_c4 == 0) {
                    unsigned long long* rec = a.records + u_rec;
                    const unsigned long long t64 = tag;
                    const unsigned long long m_bits = __builtin_bit_cast(uint32_t, mx);
                    const unsigned long long l_bits = __builtin_bit_cast(uint32_t, lsum);
                    __hip_atomic_store(rec, t64 | (m_bits << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(rec + 1, t64 | (l_bits << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            } else if (u_c4 == 0) {
                s_fin[2 * u_h] = mx;
                s_fin[2 * u_h + 1] = lsum;
            }
        }
        LLMI_STAMP(3, wave == 0);
        if (LLMI_STACK_PREFETCH_LATE) {
            while (in_flight < NSTAGE && iss_layer < sa.layers && n_my > 0) issue_next();
        }
        if (!merges_any) continue;

        // ---- (5) the log-sum-exp merge of a head's splits, one wavefront per head ----
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // its own partial stores are acknowledged
        __syncthreads();                                  // ... and its (max, sum) pairs are in LDS
        if (spread ? wave == 0 : wave < a.group) {
            const int h = spread ? merge_head : wave;
            const int c4 = lane & 31, part = lane >> 5;
            const int hq = kvh * a.group + h;
            const WsHead wh = ws_head<BYSIDE>(a, hq);
            // the records of the other splits, one per lane; this workgroup's own pair comes from LDS
            float m_reg = -INFINITY, l_reg = 0.0f;
            bool home = my_xs != 0;
            bool ok = false;
            const unsigned long long* rec_near = a.records + (int64_t)ws_row<9>(wh, min(lane, S - 1), my_xs) * 2;
            auto poll_round = [&](auto both_tag) {
                constexpr bool kBoth = decltype(both_tag)::value;
                ok = true;
                m_reg = -INFINITY;
                l_reg = 0.0f;
                if (lane < S && lane != split) {
                    const unsigned long long* rec = rec_near;
                    unsigned long long r0 = __hip_atomic_load(rec, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    unsigned long long r1 = __hip_atomic_load(rec + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    bool here = (uint32_t)r0 == tag && (uint32_t)r1 == tag;
                    if constexpr (kBoth) {
                        home = my_xs != 0;
                        if (!here) {
                            rec = a.records + (int64_t)ws_row<9>(wh, lane, my_xs ^ 1) * 2;
                            r0 = __hip_atomic_load(rec, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            r1 = __hip_atomic_load(rec + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            here = (uint32_t)r0 == tag && (uint32_t)r1 == tag;
                            home = my_xs == 0;
                        }
                    }
                    ok = here;
                    m_reg = __builtin_bit_cast(float, (uint32_t)(r0 >> 32));
                    l_reg = __builtin_bit_cast(float, (uint32_t)(r1 >> 32));
                } else if (lane == split) {
                    m_reg = s_fin[2 * h];
                    l_reg = s_fin[2 * h + 1];
                }
                return __all(ok);
            };
            constexpr int kNearRounds = 16;
            const int near_rounds = BYSIDE ? min(a.max_polls, kNearRounds) : a.max_polls;
            bool all_in = false;
            for (int spin = 0; spin < near_rounds && !all_in; ++spin) all_in = poll_round(std::false_type{});
            if constexpr (BYSIDE) {
                if (__builtin_expect(!all_in, 0)) {
                    for (int spin = near_rounds; spin < a.max_polls && !all_in; ++spin) {
                        all_in = poll_round(std::true_type{});
                        if (!all_in) __builtin_amdgcn_s_sleep(2);
                    }
                }
            }
            const bool arrived = __all(ok);
            if (__builtin_expect(!arrived, 0) && lane == 0) atomicAdd(&g_poll_timeouts, 1u);
            LLMI_STAMP(4, wave == 0);

            const uint32_t row0_bytes = (uint32_t)wh.rbase * (kHeadDim * 4u);
            const uint32_t block_mask = BYSIDE ? ~(uint32_t)(kSideBlockBytes - 1) : 0u;
            const uint32_t lane_bytes = (uint32_t)c4 * 16u;
            const bool mixed = BYSIDE && __any(home != (my_xs != 0));
            const unsigned long long home_flags = __ballot(home);
            auto load_partial = [&](int sp) {
                const int spc = min(sp, S - 1);
                const uint32_t B = row0_bytes + (uint32_t)spc * (kHeadDim * 4u);
                uint32_t home_bytes = 0u;
                if constexpr (BYSIDE) {
                    const int xs = mixed ? (int)((home_flags >> spc) & 1ull) : my_xs;
                    home_bytes = (uint32_t)(wh.ppar ^ xs) * kSideBlockBytes;
                }
                return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(part_rsrc, B + (B & block_mask) + home_bytes + lane_bytes, 0, kCacheDevice));
            };
            // lane = (16-byte column, half of the splits): all of a lane's partial rows requested at once, the weights
            // worked out while they travel
            constexpr int kBatch = 16;
            f32x4 v[kBatch];
#pragma unroll
            for (int j = 0; j < kBatch; ++j) v[j] = load_partial(part + 2 * j);
            float mx = wave_max(m_reg);
            const float f = (m_reg == -INFINITY) ? 0.0f : fast_exp2(m_reg - mx);
            float* w = s_w + h * 64;
            if (lane < S) {
                w[lane] = f;
                if (lane != split) {  // consumed: cleared, so that a replay of this launch (same tags) starts clean
                    unsigned long long* rec = a.records + (int64_t)ws_row<9>(wh, lane, home ? 1 : 0) * 2;
                    __hip_atomic_store(rec, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(rec + 1, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            const float den = wave_sum(lane < S ? l_reg * f : 0.0f);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_wave_barrier();
            f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int j = 0; j < kBatch; ++j) {
                const int sp = part + 2 * j;
                sum += v[j] * (sp < S ? w[sp] : 0.0f);
            }
            for (int s0 = part + 2 * kBatch; s0 < S; s0 += 2 * kBatch) {
#pragma unroll
                for (int j = 0; j < kBatch; ++j) v[j] = load_partial(s0 + 2 * j);
#pragma unroll
                for (int j = 0; j < kBatch; ++j) {
                    const int sp = s0 + 2 * j;
                    sum += v[j] * (sp < S ? w[sp] : 0.0f);
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) sum[e] = halves_sum(sum[e]);
            LLMI_STAMP(5, wave == 0);
            if (part == 0) {
                const float inv = (arrived && !poisoned) ? 1.0f / den : __builtin_nanf("");
                const f32x4 r = sum * inv;
                const unsigned long long packed = (unsigned long long)pack_bf16(r[0], r[1]) | ((unsigned long long)pack_bf16(r[2], r[3]) << 32);
                unsigned long long* op = reinterpret_cast<unsigned long long*>(a.out + (int64_t)layer * sa.out_stride + (int64_t)hq * kHeadDim + c4 * 4);
                // (device scope: the next layer of this launch may read this row as its query, from any XCD)
                __hip_atomic_store(op, packed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (a.out_f32) {
                    float* of = a.out_f32 + (int64_t)layer * sa.out_stride + (int64_t)hq * kHeadDim + c4 * 4;
#pragma unroll
                    for (int e = 0; e < 4; ++e) of[e] = r[e];
                }
            }
            // The head's output (and its cleared records) are acknowledged: every copy of its done tag says so.
            if (layer + 1 < sa.layers) {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                if (lane < kDoneCopies)
                    __hip_atomic_store(sa.done + (size_t)lane * words_per_copy + hq, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            LLMI_STAMP(6, wave == 0);
        }
    }
}

template <int G>
bool launch_stack_g(const StackArgs& sa, int n_kv, hipStream_t stream) {
#ifndef LLMI_STACK_WAVES
#define LLMI_STACK_WAVES 4
#endif
    constexpr int NW = LLMI_STACK_WAVES, NSTAGE = 8 / NW;  // the rings hold eight tiles per workgroup either way
    const dim3 grid(n_kv, sa.a.num_splits), block(NW * 64);
    if (sa.a.by_side) hipLaunchKernelGGL((mha_stack_kernel<G, NW, NSTAGE, true>), grid, block, 0, stream, sa);
    else hipLaunchKernelGGL((mha_stack_kernel<G, NW, NSTAGE, false>), grid, block, 0, stream, sa);
    return true;
}

}  // namespace

bool launch_stack(const StackArgs& sa, int n_kv, int group_pad, int waves, hipStream_t stream) {
    if (waves != 4) return false;  // (the plan's wave count; the kernel's own is LLMI_STACK_WAVES)
    switch (group_pad) {
        case 1: return launch_stack_g<1>(sa, n_kv, stream);
        case 2: return launch_stack_g<2>(sa, n_kv, stream);
        case 4: return launch_stack_g<4>(sa, n_kv, stream);
        default: return false;
    }
}

size_t stack_done_bytes(int head_num) {
    return (size_t)kDoneCopies * (size_t)((head_num + kDoneLineWords - 1) / kDoneLineWords) * kDoneLineWords * sizeof(uint32_t);
}

hipError_t poll_timeouts_stack(unsigned int* n) { return hipMemcpyFromSymbol(n, HIP_SYMBOL(g_poll_timeouts), sizeof(*n)); }

}  // namespace llmi
