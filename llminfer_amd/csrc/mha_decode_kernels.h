// Decode-phase grouped-query attention for gfx950 (MI355X), batch 1: the kernel templates.
// Included by one translation unit per query-group size (mha_decode_group*.hip defines LLMI_GROUP first), which
// instantiates the kernels of that group; the host-side launcher is mha_decode.hip.
//
// One kernel template serves both paths of the reference's dispatcher
// (code/source/op/kernel/cuda/mha_kernel.cu:505-528):
//   * single pass  (num_splits == 1): the workgroup owns every position of one
//     KV head and writes the bf16 result itself;
//   * KV split     (num_splits  > 1): workgroup (split, kv_head) owns a
//     contiguous range of positions and leaves (o[128], m, l) per query head
//     in the fp32 workspace; either mha_combine_kernel merges them
//     (log-sum-exp, a second launch) or the workgroup of the last split does,
//     inside the same launch (fused combine).
// Three more template switches: APPEND folds the per-token QK-Norm + RoPE and the
// K/V cache append of the reference's layer loop into the launch (the new row
// enters the softmax from registers), DYN reads the position from device memory
// so that one captured launch serves every token, STAGGER makes the splits of the
// position-major layout walk their tiles from different starting points.
//
// Differences from the reference design, chosen for CDNA4:
//   * a workgroup serves ALL query heads of its KV head, so K and V are read
//     from HBM exactly once (the reference re-reads them once per query head,
//     mha_kernel.cu:67,104);
//   * K/V tiles stream through per-wave LDS rings filled by LDS-DMA loads, every
//     load instruction a run of whole 256-byte rows (1 KiB of contiguous memory
//     in the head-major layout); the query rows (and the append variant's operands)
//     take the same road, issued ahead of the tiles, so that every wait is a hand-placed vmcnt;
//   * q.K^T runs on the matrix cores: one v_mfma_f32_16x16x32_bf16 chain per
//     tile of 16 positions, K rows as the A operand (lane = row, no transpose
//     needed because the contraction over head_dim is order-free), the query
//     group as B;
//   * P^T.V runs on the matrix cores too (v_mfma_f32_16x16x16_bf16): the score
//     MFMA leaves a lane's four probabilities exactly where the A fragment of
//     that product wants them, the V fragment is packed from the lane's four
//     16-byte V rows with v_perm_b32; a probability enters as hi + lo bf16, so
//     the product is as accurate as an fp32 one;
//   * running max / sum are kept in the exp2 domain (scale*log2(e) folded in);
//   * 64-bit offsets throughout (the reference's int32 layer_offset,
//     mha_kernel.cu:488, overflows on large caches).
//
// Tile bookkeeping (T = 16 consecutive positions, r = row in tile, h = head in group):
//   QK  A  lane L: row r = L%16, dims (j*4 + L/16)*8 .. +8 for step j = 0..3
//   QK  B  lane L: head h = L%16 (zero for h >= group), same dims
//   QK  C  lane L: head h = L%16, rows r = 4*(L/16) + i in register i = 0..3
//   loads  lane L: K and V load i fetch rows 4i + L/16 whole (256 contiguous bytes over the row's 16 lanes;
//                  K with its 16-byte chunks swizzled by row & 7); the operands are read back from
//                  LDS in the layouts above and below
//   V oper lane L: rows r = 4*(L/16) + i (register i), columns (L%16)*8 .. +8
//   PV  A  lane L: head h = L%16, rows 4*(L/16) + i      (= QK C, as bf16)
//   PV  B  lane L: rows 4*(L/16) + i, column 8*(L%16) + j for product j = 0..7
//   PV  C  lane L: heads 4*(L/16) + i, column 8*(L%16) + j (accumulator o[j][i])

#ifndef LLMI_MHA_DECODE_KERNELS_H
#define LLMI_MHA_DECODE_KERNELS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "mha_device_helpers.h"

namespace llmi {
namespace {

// Occupancy hint. Two waves per SIMD keep the register budget at 256, where the compiler picks
// VGPR-form MFMAs; with the whole file of 512 it keeps the accumulators in AGPRs and copies them to
// VGPRs and back around the rescaling of every tile. Groups of 16 heads cannot meet the hint in every
// shape; there it is 1.
template <int G, int NW>
constexpr int kWavesPerEu = (G >= 16 && NW != 2) ? 1 : LLMI_MIN_WAVES_PER_EU;

template <int G, int NW, int NSTAGE, bool APPEND, bool DYN, bool STAGGER, bool OPROJ, bool BYSIDE>
__device__ __forceinline__ void mha_decode_body(const KernelArgs& a, OprojState& proj) {
    constexpr bool kSpreadMerge = LLMI_SPREAD_MERGE && !OPROJ && G <= NW;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: loop control stays on the SALU
    const int n16 = lane & 15;  // MFMA column / DPP-row lane
    const int kg = lane >> 4;   // MFMA k-group / DPP row
    // Workgroups are handed to the eight XCDs (each with its own L2) in turn, in index order with x
    // fastest: with the KV head in x, the splits of a head land on one XCD whenever the number of
    // KV heads is a multiple of eight, and the combiners (last splits) spread over all of them
    // instead of sharing one. Nothing relies on that placement for correctness; it is worth
    // 0.1-0.35 us per call (32 query / 8 KV heads, 1K to 32K positions) against split-fastest.
    const int kvh = blockIdx.x;
    const int split = blockIdx.y;

    // A KV head's 16-position tiles are dealt to the splits in contiguous runs whose lengths
    // differ by at most one tile (the first tiles % S splits get the longer run), so every split
    // has work whenever there are at least S tiles and the last split -- the one that merges,
    // and in the append variant the one that holds the new token -- never has the longest run.
    // With a position read from device memory the grid was sized for the largest position:
    // the same rule is applied to the tiles there are, and splits beyond the tile count leave
    // at once.
    // Append variant: the new token's row never comes from the cache (its K and V are in registers
    // and go straight into the running softmax of one wave), so the tiles cover positions 0 .. pos-1.
    int seq_len = a.seq_len, n_active = a.num_splits;
    if constexpr (DYN) {
        seq_len = max(0, min(*a.pos_dev, a.seq_len - 1)) + 1;
        n_active = min(a.num_splits, max(1, (seq_len - (APPEND ? 1 : 0) + kTile - 1) / kTile));
        if (split >= n_active) return;
    }
    const int cached_len = seq_len - (APPEND ? 1 : 0);  // positions streamed from the cache
    // (the host never asks for more splits than tiles; 0 tiles: 1 split). The division is done on
    // the host when the position is known there: it is 33 instructions in front of the first load.
    int run = a.tiles_run, longer = a.tiles_longer;  // splits 0 .. longer-1 take run + 1 tiles
    if constexpr (DYN) {
        const int total_tiles = (cached_len + kTile - 1) / kTile;
        run = total_tiles / n_active;
        longer = total_tiles % n_active;
    }
    const int ntiles = run + (split < longer ? 1 : 0);
    const int begin = (split * run + min(split, longer)) * kTile;
    const int nrows = min(ntiles * kTile, cached_len - begin);  // > 0 unless nothing is cached yet

    // Filled in below, once the first tiles are on their way.
    u32x4 qb[4];                       // query group, MFMA B operand
    // Append variant: wave 0 of the last split (the one with the shortest run) takes the new token.
    const bool holds_new_row = APPEND && split == n_active - 1 && wave == 0;

    // Wave-uniform 64-bit bases of this split; lanes add 32-bit byte offsets
    // (scalar-base + vector-offset addressing, no 64-bit multiplies per load).
    const char* kb = reinterpret_cast<const char*>(a.k + (int64_t)kvh * a.head_stride + (int64_t)begin * a.row_stride);
    const char* vb = reinterpret_cast<const char*>(a.v + (int64_t)kvh * a.head_stride + (int64_t)begin * a.row_stride);
    const uint32_t rs = (uint32_t)a.row_stride * 2u;           // bytes per position step
    const uint32_t last_off = (uint32_t)(nrows - 1) * rs;      // rows past the range clamp to its last row
    // K load i of a tile fetches rows 4i .. 4i+3 whole (DPP row kg takes row 4i + kg, 256 contiguous
    // bytes across its 16 lanes): every request is a full cache line in either layout, and in the
    // head-major layout one instruction covers 1 KiB of contiguous memory. Lane p of the row fetches
    // 16-byte chunk p ^ (row & 7): the swizzle that lets the MFMA operand read below (lane = row,
    // 16 rows 256 bytes apart) spread over the LDS banks instead of hitting one.
    const uint32_t k_row = (uint32_t)kg * rs;
    const uint32_t k_col0 = (uint32_t)(n16 ^ kg) * 16u;        // rows 4i + kg with i even: (row & 7) = kg
    const uint32_t k_col1 = (uint32_t)(n16 ^ (4 + kg)) * 16u;  // i odd: (row & 7) = 4 + kg
    // Operand read: row n16 sits in load n16 / 4, at row slot n16 % 4; chunk c is at lane slot c ^ (n16 & 7).
    const uint32_t k_rd = (uint32_t)((n16 >> 2) * 1024 + (n16 & 3) * 256);
    const uint32_t k_rd0 = k_rd + (uint32_t)((kg ^ (n16 & 7)) * 16);        // chunks j*4 + kg, j even (+ 128 bytes for j = 2)
    const uint32_t k_rd1 = k_rd + (uint32_t)(((4 + kg) ^ (n16 & 7)) * 16);  // j odd (+ 128 bytes for j = 3)
    const uint32_t v_col = (uint32_t)n16 * 16u;

    float m_run = -INFINITY;  // running max, exp2 domain, per (head = n16)
    float l_run = 0.0f;       // running sum over this lane's rows
    // Output accumulators, MFMA C layout of P^T V: o[j][r] belongs to head 4*kg + r and
    // column 8*n16 + j, summed over all positions this wave has seen.
    f32x4 o[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#if LLMI_PV_VALU
    // Vector-ALU variant: ov[h][j] belongs to head h and column 8*n16 + j, summed over the rows
    // 4*kg .. 4*kg+3 of every tile this wave has seen; the four DPP rows are added up after the loop.
    float ov[G][8];
#pragma unroll
    for (int h = 0; h < G; ++h)
#pragma unroll
        for (int j = 0; j < 8; ++j) ov[h][j] = 0.0f;
#endif

    // Each wave streams its tiles through a private ring of NSTAGE LDS slots
    // (8 KiB each: 4 KiB of K rows, 4 KiB of V rows) filled by LDS-DMA loads,
    // so the bytes in flight cost no VGPRs. A load lands at offset 16*lane of its
    // 1 KiB block, i.e. as four whole rows; the operand reads pick their 16 bytes
    // out of those rows (K through a row-dependent swizzle, V directly), both free
    // of bank conflicts. Out-of-range rows of a ragged last
    // tile read the last valid row and are masked out of the softmax.
    constexpr int kStageBytes = 8192;
    constexpr int kRingBytes = NW * NSTAGE * kStageBytes;
    // Epilogue: a wave's G x 128 partial outputs go to the start of its own (drained) ring,
    // so no wave has to wait for another one's ring. Behind the rings: per-wave and merged
    // (max, sum) pairs, then the combine area (weights [G][kMaxSplits], denominators [G],
    // per-wave arrival flags [NW], one 16-byte partial sum per thread).
    constexpr int kWaveRingBytes = NSTAGE * kStageBytes;
    static_assert(G * kHeadDim * (int)sizeof(float) <= kWaveRingBytes, "a wave's partial outputs must fit its ring");
    constexpr int kMergeTail = (2 * NW * G + 2 * G) * (int)sizeof(float);
    constexpr int kCombineBase = kRingBytes + ((kMergeTail + 15) & ~15);
    constexpr int kCombineBytes = (G * kMaxSplits + G + NW) * (int)sizeof(float) + NW * 64 * 16;
    // 1 KiB LDS-DMA slots for the small operands. Per wave: the query rows of the group (16 chunks
    // of 16 bytes per head, four heads to a slot; normalised in place in the append variant).
    // Append variant, in front of them and shared by the workgroup (every wave fills them with
    // the same bytes and waits only for its own loads): slot 0 = q_norm | k_norm | sin row |
    // cos row, 16 chunks each; slot 1 = new K row | new V row, used by one wave only. The slots
    // lie over the combine area, which nobody touches before the barrier of the epilogue, so they
    // cost no LDS: with more than 80 KiB per workgroup the compiler assumes one wave per SIMD, puts
    // the MFMA accumulators into AGPRs and copies all 32 of them to VGPRs and back around the
    // rescaling of every tile.
    constexpr int kQSlots = (G * 16 + 63) / 64;
    constexpr int kSharedSlots = APPEND ? 2 : 0;
    constexpr int kStagingBase = (kCombineBase + 1023) & ~1023;
    constexpr int kStagingBytes = (kSharedSlots + NW * kQSlots) * 1024;
    constexpr int kSmemBytes =
        kCombineBase + kCombineBytes > kStagingBase + kStagingBytes ? kCombineBase + kCombineBytes : kStagingBase + kStagingBytes;
    __shared__ __attribute__((aligned(1024))) char smem[kSmemBytes];
    char* my_ring = smem + wave * (NSTAGE * kStageBytes);
    const uint32_t my_ring_lds = (uint32_t)(uintptr_t)my_ring;  // low 32 bits of a flat LDS address = LDS offset

    auto issue_tile = [&](int t, int stage) {
        // The slot's previous contents must have reached the VGPRs first.
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        const uint32_t base = (uint32_t)t * (kTile * rs);
        const uint32_t slot = my_ring_lds + (uint32_t)stage * kStageBytes;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t ko = min(base + k_row + (uint32_t)(4 * i) * rs, last_off) + ((i & 1) ? k_col1 : k_col0);
            dma16(kb, ko, slot + i * 1024);
        }
        // V the same way: load i fetches rows 4i .. 4i+3 whole. The operand wants rows 4*kg + i in lane
        // (kg, n16): row r sits in load r / 4 at row slot r % 4, read back below without bank conflicts
        // (the 16 lanes of a DPP row read 256 consecutive bytes).
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t vo = min(base + k_row + (uint32_t)(4 * i) * rs, last_off) + v_col;
            dma16(vb, vo, slot + 4096 + i * 1024);
        }
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

    auto compute_tile = [&](int t, const TileRegs& r) {
        f32x4 c = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < 4; ++j)
            c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, r.k[j]),
                                                        __builtin_bit_cast(bf16x8, qb[j]), c, 0, 0, 0);
        const int row0 = t * kTile + 4 * kg;
        float s[4];
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            s[i] = (row0 + i < nrows) ? c[i] * a.scale_log2e : -INFINITY;
            tmax = fmaxf(tmax, s[i]);
        }
        tmax = rows_max(tmax);
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = fast_exp2(m_run - m_new);
        float p[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) p[i] = fast_exp2(s[i] - m_new);
        const float psum = (p[0] + p[1]) + (p[2] + p[3]);
        l_run = l_run * alpha + psum;
        m_run = m_new;
#if LLMI_PV_VALU
        // Rescale only when some head's max moved (wave-uniform test); head h's factor sits in
        // lane h of every 16-lane row.
        if (__any(alpha != 1.0f)) {
            static_for<0, G>([&](auto h) {
                const float ah = row_bcast<h.value>(alpha);
#pragma unroll
                for (int j = 0; j < 8; ++j) ov[h.value][j] *= ah;
            });
        }
        float vf[4][8];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t w = r.v[i][j >> 1];
                vf[i][j] = (j & 1) ? bf16_hi(w) : bf16_lo(w);
            }
        static_for<0, G>([&](auto h) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float ph = row_bcast<h.value>(p[i]);  // probability of (head h, row 4*kg + i)
#pragma unroll
                for (int j = 0; j < 8; ++j) ov[h.value][j] = fmaf(ph, vf[i][j], ov[h.value][j]);
            }
        });
#else
        // The probabilities enter the second MFMA as a sum of two bf16 numbers
        // (p = hi + lo, relative error 2^-17), so that the product keeps fp32-like accuracy.
        const uint32_t p01 = pack_bf16(p[0], p[1]);
        const uint32_t p23 = pack_bf16(p[2], p[3]);
        const uint32_t q01 = pack_bf16(p[0] - bf16_lo(p01), p[1] - bf16_hi(p01));
        const uint32_t q23 = pack_bf16(p[2] - bf16_lo(p23), p[3] - bf16_hi(p23));

        // Rescale only when some head's max moved (wave-uniform test). The factor of
        // head 4*kg + r sits in lane 4*kg + r of this lane's 16-lane row.
        if (__any(alpha != 1.0f)) {
            static_for<0, 4>([&](auto r) {
                float ar;
                if constexpr (G <= 4) ar = row_bcast<r.value>(alpha);  // only row kg = 0 holds heads
                else ar = row_bcast_per_row<r.value>(alpha);           // DPP row k takes lane 4*k + r of its own row
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j][r.value] *= ar;
            });
        }
        // O^T += P^T V on the matrix cores: A = P^T (head x position: this lane's four
        // probabilities are exactly its A fragment), B = V (position x column, column
        // 8*n + j for output lane n: element j of each of the lane's four V rows).
        const i16x4 pa = __builtin_bit_cast(i16x4, u32x2{p01, p23});
        const i16x4 pb = __builtin_bit_cast(i16x4, u32x2{q01, q23});
        i16x4 vb[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;  // high or low halves
            const uint32_t b01 = __builtin_amdgcn_perm(r.v[1][j >> 1], r.v[0][j >> 1], sel);
            const uint32_t b23 = __builtin_amdgcn_perm(r.v[3][j >> 1], r.v[2][j >> 1], sel);
            vb[j] = __builtin_bit_cast(i16x4, u32x2{b01, b23});
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(pa, vb[j], o[j], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(pb, vb[j], o[j], 0, 0, 0);
#endif
    };

    // Wave w owns tiles w, w+NW, ...: NSTAGE of them are always in flight.
    const int n_my = wave < ntiles ? (ntiles - wave + NW - 1) / NW : 0;
    // STAGGER: the splits of a head walk their tiles from different starting points (split s starts
    // s & a.stagger tiles into its wave's sequence and wraps round), so that workgroups running in
    // step do not all sit at the same offset of their runs. Where the runs start a multiple of 512 KiB
    // apart, walking them in step keeps hitting the same few memory channels: position-major, 8192
    // positions, 1.7 us of 13.6; head-major, 131072 positions (runs of 1 MiB), up to 6 us of 86. Elsewhere it
    // gains nothing or loses, and the bookkeeping costs 0.08 us per call, so the host asks for it by
    // length and it is compiled in only where it is used.
    // (position read on the device: the host could only say that the rule may apply; what the length found asks for)
    int rot_mask = a.stagger;
    if constexpr (DYN && STAGGER)
        if (rot_mask == kStaggerByDevice) rot_mask = head_major_stagger_rule((long long)run * kTile * a.row_stride * 2);
    const int rot = STAGGER ? min(split & rot_mask, max(n_my - 1, 0)) : 0;
    auto tile_of = [&](int i) {
        if constexpr (!STAGGER) return wave + i * NW;
        int ii = i + rot;
        if (ii >= n_my) ii -= n_my;
        return wave + ii * NW;
    };
    // The query rows (and in the append variant the operands of the fused QK-Norm + RoPE) go to
    // LDS by DMA *ahead of* the first K/V tiles. Loads complete in order, so they are there
    // after one memory round trip: the normalisation runs while the tiles are still in flight,
    // and the first tile is worked on as soon as it lands. As ordinary loads their wait would be
    // placed by the compiler, which does not know about the DMA loads: it would also wait for
    // every tile issued before that point.
    if constexpr (OPROJ) {
        // The generation word moves once per launch, after every head's output is written. That needs
        // every combiner, each combiner needs the records of its splits, and those go out only after
        // every load of this wavefront has come back (the wait in front of the record stores): read
        // here, the word still holds the value of before, in every workgroup of the grid. Issued ahead of
        // the tiles, so that nothing near the end of the kernel has to wait for it.
        proj.gen_base = __hip_atomic_load(a.ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    char* shared_staging = smem + kStagingBase;                                     // append variant only
    char* my_rows = smem + kStagingBase + (kSharedSlots + wave * kQSlots) * 1024;  // this wave's query rows
    {
        const uint32_t st = (uint32_t)(uintptr_t)shared_staging;
        const uint32_t st_rows = (uint32_t)(uintptr_t)my_rows;
        const int c16 = lane & 15, which = lane >> 4;
        if constexpr (APPEND) {
            const float* sin_row = a.sin_cache + (int64_t)(seq_len - 1) * 64;
            const float* cos_row = a.cos_cache + (int64_t)(seq_len - 1) * 64;
            // (integer selects: as pointer conditionals this becomes a chain of branches)
            const uint64_t w_base = reinterpret_cast<uint64_t>(a.norm_w) + (uint64_t)(which & 1) * 256u;
            const uint64_t t_base = reinterpret_cast<uint64_t>(which == 2 ? sin_row : cos_row);
            const uint64_t p0 = (which < 2 ? w_base : t_base) + (uint64_t)c16 * 16u;
            dma16_gather(reinterpret_cast<const void*>(p0), st);
            if (holds_new_row) {
                const uint64_t p1 = reinterpret_cast<uint64_t>((which & 1) == 0 ? a.k_new : a.v_new) +
                                    (uint64_t)(kvh * kHeadDim * 2 + c16 * 16);
                dma16_gather(reinterpret_cast<const void*>(p1), st + 1024);
            }
        }
#pragma unroll
        for (int i = 0; i < kQSlots; ++i) {
            const int head = min(which + 4 * i, a.group - 1);  // chunk lane + 64*i: head (lane + 64*i) / 16
            dma16_gather(a.q + (int64_t)(kvh * a.group + head) * kHeadDim + c16 * 8, st_rows + i * 1024);
        }
    }
#pragma unroll
    for (int s0 = 0; s0 < NSTAGE; ++s0)
        if (s0 < n_my) issue_tile(tile_of(s0), s0);
    // What the end of the kernel needs to know about where its results go is worked out here, while the first tiles
    // are on their way and the wavefront has nothing else to do: behind the last tile every instruction is on the
    // path of whoever waits for this split (the empty asm statements keep the compiler from moving the work there).
    const bool fused = a.records != nullptr && n_active > 1;
    const int my_xs = package_side<BYSIDE>();  // wave-uniform: the side of the package this workgroup runs on
    // Who merges a query head's splits (log-sum-exp): where one wavefront merges a head (G <= NW) and there are at
    // least as many splits as heads in the group, head h's splits are merged by wavefront 0 of the workgroup of split
    // SA-1-h, so that the heads' read-backs (16 KiB each at 32 splits) run on different compute units at the same
    // time instead of queueing at one; otherwise the workgroup of the last split merges every head.
    const bool spread = kSpreadMerge && a.spread_merge && n_active >= a.group;
    const int merge_head = spread && n_active - 1 - split < a.group ? n_active - 1 - split : -1;
    const bool merges_any = spread ? merge_head >= 0 : split == n_active - 1;
    // (testing aid: pretend this split ran on the other side; never a merging one, whose own rows it reads itself)
    const int store_xs = my_xs ^ (int)(BYSIDE && !merges_any && (a.far_home == 1 || (a.far_home == 2 && (split & 1))));
    const int n_units = a.group * (kHeadDim / 4);
    const int64_t part_rows = BYSIDE ? 2 * (((int64_t)a.n_q * a.num_splits + 15) & ~(int64_t)15) : (int64_t)a.n_q * a.num_splits;
    int part_bytes = (int)(part_rows * kHeadDim * (int64_t)sizeof(float));
    asm volatile("" : "+s"(part_bytes));
    const __amdgpu_buffer_rsrc_t part_rsrc = __builtin_amdgcn_make_buffer_rsrc(a.ws, 0, part_bytes, 0x00020000);
    // A (head, 16-byte column) unit of the final merge: where its partial row and its record go.
    struct MergeUnit {
        int hq;
        int64_t po;               // element offset of the column in the partial array
        int64_t rec;              // index of the first word of the head's record of this split (fused combine)
    };
    auto merge_unit = [&](int u) {
        const int h = u >> 5, c4 = u & 31;
        MergeUnit m;
        m.hq = kvh * a.group + h;
        const WsHead wh = ws_head<BYSIDE>(a, m.hq);
        m.po = (fused ? (int64_t)ws_row<4>(wh, split, store_xs) : (int64_t)m.hq * a.num_splits + split) * kHeadDim + c4 * 4;
        m.rec = (int64_t)ws_row<9>(wh, split, store_xs) * 2;
        return m;
    };
    MergeUnit first_unit = merge_unit((int)threadIdx.x);
    asm volatile("" : "+v"(first_unit.hq), "+v"(first_unit.po), "+v"(first_unit.rec));
    // Query group as the MFMA B operand (zero columns beyond the group; rows beyond it
    // were filled with copies of its last row).
    {
        // Everything issued before the tiles has landed once only the tiles are in flight.
        wait_tiles_in_flight(min(NSTAGE, n_my));
        const u32x4* sh4 = reinterpret_cast<const u32x4*>(shared_staging);
        const u32x4* rows4 = reinterpret_cast<const u32x4*>(my_rows);
        if constexpr (APPEND) {
            // Four rows at a time, one per DPP row.
#pragma unroll
            for (int b4 = 0; b4 < kQSlots; ++b4)
                norm_rope_rows_lds(my_rows, shared_staging, shared_staging + 512, shared_staging + 768, 4 * b4 + kg, n16, a.eps);
            if (holds_new_row)  // the new K row: all four DPP rows work on the one row
                norm_rope_rows_lds(shared_staging + 1024, shared_staging + 256, shared_staging + 512, shared_staging + 768, 0, n16,
                                   a.eps);
        }
        const int hq_local = min(n16, a.group - 1);
        const bool live = n16 < a.group;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const u32x4 qv = rows4[hq_local * 16 + j * 4 + kg];
            qb[j] = live ? qv : u32x4{0u, 0u, 0u, 0u};
        }
        // Fused append: this wave files the new token's K row (normalised + rotated above) and V
        // row in the cache and starts its running softmax from that one position -- score q.k,
        // weight 1, output = the V row -- while its first tiles are still on their way.
        if constexpr (APPEND) {
            if (holds_new_row) {
                typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
                u32x4 kf[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) kf[j] = sh4[64 + j * 4 + kg];  // operand layout, as a K row of a tile
                const u32x4 vf = sh4[64 + 16 + n16];                          // columns 8*n16 .. +7
                if (n16 == 0) {
                    uint16_t* kd = const_cast<uint16_t*>(a.k) + (int64_t)(seq_len - 1) * a.row_stride + kvh * a.slot_head_stride;
#pragma unroll
                    for (int j = 0; j < 4; ++j) *reinterpret_cast<u32x4*>(kd + (j * 4 + kg) * 8) = kf[j];
                }
                if (kg == 0)
                    *reinterpret_cast<u32x4*>(const_cast<uint16_t*>(a.v) + (int64_t)(seq_len - 1) * a.row_stride +
                                              kvh * a.slot_head_stride + n16 * 8) = vf;
                float dot = 0.0f;
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const uint32_t qw = qb[j][c], kw = kf[j][c];  // (bit_cast straight from a vector element reads element 0)
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
#if LLMI_PV_VALU
#pragma unroll
                    for (int h = 0; h < G; ++h) ov[h][j] = kg == 0 ? vj : 0.0f;
#endif
                }
            }
        }
    }

    int stage = 0;
#if LLMI_TIMING_BARRIER_PER_TILE
    // (measurement only: what a scheme in which the wavefronts of a workgroup share every tile would pay for having to
    // agree, tile by tile, that a slot may be refilled -- a workgroup barrier per tile, every wavefront the same number)
    for (int i = 0; i < (ntiles + NW - 1) / NW; ++i) {
        __syncthreads();
        if (i >= n_my) continue;
#else
    for (int i = 0; i < n_my; ++i) {
#endif
        TileRegs r;
        wait_tiles_in_flight(min(NSTAGE - 1, n_my - 1 - i));
        read_tile(stage, r);
        if (i + NSTAGE < n_my) issue_tile(tile_of(i + NSTAGE), stage);
        compute_tile(tile_of(i), r);
        stage = (stage + 1 == NSTAGE) ? 0 : stage + 1;
    }

    // ---- epilogue: fold the workgroup's waves ----
    // The outputs are already summed over a wave's positions; the denominators are
    // per DPP row (kg) and share the running max of their head, so they add up plainly.
    l_run = rows_sum(l_run);
#if LLMI_PV_VALU
    // Into the layout the epilogue expects: o[j][r] of DPP row kg is head 4*kg + r.
    static_for<0, G>([&](auto h) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float t = rows_sum(ov[h.value][j]);
            if (kg == h.value / 4) o[j][h.value % 4] = t;
        }
    });
#endif

    // This wave's ring is drained (every tile it issued was waited for and read).
    typedef float (*MergeS)[G];
    auto s_o = [&](int w, int h) { return reinterpret_cast<float*>(smem + w * kWaveRingBytes) + h * kHeadDim; };
    MergeS s_m = reinterpret_cast<MergeS>(smem + kRingBytes);
    MergeS s_l = s_m + NW;
    float* s_fin = reinterpret_cast<float*>(s_l + NW);  // [G][2]: merged (max, sum) per head
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int h = 4 * kg + r;
        if (h < G) {
            float* dst = s_o(wave, h) + n16 * 8;
            *reinterpret_cast<f32x4*>(dst) = f32x4{o[0][r], o[1][r], o[2][r], o[3][r]};
            *reinterpret_cast<f32x4*>(dst + 4) = f32x4{o[4][r], o[5][r], o[6][r], o[7][r]};
        }
    }
    if (kg == 0 && n16 < G) {
        s_m[wave][n16] = m_run;
        s_l[wave][n16] = l_run;
    }
    __syncthreads();

    if constexpr (OPROJ) proj.worker = split != n_active - 1;
    // One thread per (head, 16-byte column): weights e^(m_w - M) of the waves, weighted sum.
    for (int u = threadIdx.x; u < n_units; u += NW * 64) {
        const int h = u >> 5;
        const int c4 = u & 31;
        MergeUnit unit = first_unit;  // (worked out while the first tiles were on their way)
        if (u != (int)threadIdx.x) unit = merge_unit(u);
        // (all of a unit's LDS reads are requested before the first is used: one round trip, not two)
        float mw[NW], lw[NW];
        f32x4 ow[NW];
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            mw[w] = s_m[w][h];
            lw[w] = s_l[w][h];
            ow[w] = *reinterpret_cast<const f32x4*>(s_o(w, h) + c4 * 4);
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
        const int hq = unit.hq;
        if (n_active == 1) {
            const f32x4 r = acc * (1.0f / lsum);  // (one division, like the fused combine's)
            *reinterpret_cast<uint2*>(a.out + (int64_t)hq * kHeadDim + c4 * 4) = make_uint2(pack_bf16(r[0], r[1]), pack_bf16(r[2], r[3]));
            if (a.out_f32) {
                float* of = a.out_f32 + (int64_t)hq * kHeadDim + c4 * 4;  // only 4-byte alignment is promised
#pragma unroll
                for (int e = 0; e < 4; ++e) of[e] = r[e];
            }
        } else {
            const int64_t S = a.num_splits;
            const int64_t po = unit.po;  // element offset in the workspace
            if (fused) {
                // Device-coherent store (cache policy sc1): it goes past this XCD's L2, so the
                // workgroup (possibly on another XCD) that does the combine can read it without
                // anyone flushing or invalidating a cache.
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc), part_rsrc,
                                                       (uint32_t)(po * (int64_t)sizeof(float)), 0, 16);
                if (spread ? h != merge_head : split != n_active - 1) {
                    // Publish the head's record as soon as this wavefront's stores are acknowledged:
                    // the 32 columns of a head are stored by one half of one wavefront, so no
                    // workgroup barrier is needed.
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    if (c4 == 0) {
                        unsigned long long* rec = a.records + unit.rec;
                        const unsigned long long tag = a.tag;
                        const unsigned long long m_bits = __builtin_bit_cast(uint32_t, mx);
                        const unsigned long long l_bits = __builtin_bit_cast(uint32_t, lsum);
                        __hip_atomic_store(rec, tag | (m_bits << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(rec + 1, tag | (l_bits << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                } else if (c4 == 0) {  // the workgroup that merges this head keeps its own pair in LDS
                    s_fin[2 * h] = mx;
                    s_fin[2 * h + 1] = lsum;
                }
            } else {
                *reinterpret_cast<f32x4*>(a.ws + po) = acc;
                if (c4 == 0) {
                    a.ws[(int64_t)a.n_q * S * kHeadDim + (int64_t)hq * S + split] = mx;
                    a.ws[(int64_t)a.n_q * S * (kHeadDim + 1) + (int64_t)hq * S + split] = lsum;
                }
            }
        }
    }
    if (!fused) return;

    // ---- fused combine ----
    // The workgroup of the LAST split of this KV head merges the partials of its
    // query heads, so no second launch is needed. Every split publishes, per query
    // head, a record {epoch | max} {epoch | sum} as soon as the head's partial outputs have
    // been acknowledged; the last split's workgroup waits for all records but its own (it
    // has its own pair in LDS and its own partials acknowledged). Workgroups are
    // dispatched in index order and the others never wait for anything, so whoever
    // it waits for is already running or done.
    // A record carries the epoch of the call that wrote it; anything else (an
    // uninitialised workspace, an earlier call) reads as "not arrived", so the
    // workspace needs no clearing. The combiner zeroes the records again so that a
    // graph replay of this very call (same epoch) starts clean.
    const int S = a.num_splits;  // layout stride of partials and records
    const int SA = n_active;     // splits that hold positions
    if (!merges_any) return;  // (its records went out above)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the combiner's own partial stores are acknowledged
    __syncthreads();                                  // ... and its (max, sum) pairs are in LDS

    float* s_w = reinterpret_cast<float*>(smem + kCombineBase);  // [G][kMaxSplits] weights
    float* s_den = s_w + G * kMaxSplits;                         // [G] denominators
    int* s_ok = reinterpret_cast<int*>(s_den + G);               // [NW] every record seen
    f32x4* s_part = reinterpret_cast<f32x4*>(s_ok + NW);         // [NW * 64] per-thread partial sums
    // Waits for the records of head h (one wavefront does); the (max, sum) pairs stay in the polling
    // lanes' registers. This workgroup's own pair comes straight from LDS: its record would be the
    // last one to become visible. Returns false if a record never came. A record only counts when
    // it carries this call's tag (never zero, which is what a cleared record holds).
    auto wait_records = [&](int h, auto slots, float* m_reg, float* l_reg, bool* home) -> bool {
        constexpr int kSlots = decltype(slots)::value;  // splits per lane
#pragma unroll
        for (int j = 0; j < kSlots; ++j) {
            m_reg[j] = -INFINITY;
            l_reg[j] = 0.0f;
            home[j] = my_xs != 0;  // the side whose home a split's record was found in: its partial outputs are in that side's home too
        }
        bool ok = false;
        // Bounded wait: every wave leaves this loop even if a record never shows up
        // (the result is then poisoned below instead of hanging the GPU).
        const WsHead wh = ws_head<BYSIDE>(a, kvh * a.group + h);
        const unsigned long long* rec_near[kSlots];
#pragma unroll
        for (int j = 0; j < kSlots; ++j) rec_near[j] = a.records + (int64_t)ws_row<9>(wh, min(lane + 64 * j, SA - 1), my_xs) * 2;
        // One round of polls. BOTH: also look where a split that ran on the other side of the package would have put its
        // record (never needed when the workgroups of a KV head share an XCD, so the first rounds do without).
        auto poll_round = [&](auto both_tag) {
            constexpr bool kBoth = decltype(both_tag)::value;
            ok = true;
#pragma unroll
            for (int j = 0; j < kSlots; ++j) {
                const int sp = lane + 64 * j;
                m_reg[j] = -INFINITY;
                l_reg[j] = 0.0f;
                if (sp < SA && sp != split) {
                    const unsigned long long* rec = rec_near[j];
                    unsigned long long r0 = __hip_atomic_load(rec, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    unsigned long long r1 = __hip_atomic_load(rec + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    bool here = (uint32_t)r0 == a.tag && (uint32_t)r1 == a.tag;
                    if constexpr (kBoth) {
                        home[j] = my_xs != 0;
                        if (!here) {
                            rec = a.records + (int64_t)ws_row<9>(wh, sp, my_xs ^ 1) * 2;
                            r0 = __hip_atomic_load(rec, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            r1 = __hip_atomic_load(rec + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            here = (uint32_t)r0 == a.tag && (uint32_t)r1 == a.tag;
                            home[j] = my_xs == 0;
                        }
                    }
                    ok = ok && here;
                    m_reg[j] = __builtin_bit_cast(float, (uint32_t)(r0 >> 32));
                    l_reg[j] = __builtin_bit_cast(float, (uint32_t)(r1 >> 32));
                } else if (sp == split) {
                    m_reg[j] = s_fin[2 * h];
                    l_reg[j] = s_fin[2 * h + 1];
                }
            }
            return __all(ok);
        };
        // The first rounds poll the near home only (some ten microseconds: far beyond the spread of the splits).
        constexpr int kNearRounds = 16;
        const int near_rounds = BYSIDE ? min(a.max_polls, kNearRounds) : a.max_polls;
        bool all_in = false;
        // (back to back: a round is one round trip of the memory system; a pause between rounds only adds to the
        // wait -- 0.03-0.06 us per call with s_sleep 2, measured at every length)
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
        // A give-up is counted where the host can read it (llmi_hip_poll_timeouts).
        if (__builtin_expect(!arrived, 0) && lane == 0) atomicAdd(&g_poll_timeouts, 1u);
        return arrived;
    };
    // From the polled (max, sum) pairs: M = max m_s, the weights e^(m_s - M) into the head's row
    // of s_w, the denominator sum l_s * weight; the records are zeroed for the next use.
    auto make_weights = [&](int h, auto slots, const float* m_reg, const float* l_reg, const bool* home) -> float {
        constexpr int kSlots = decltype(slots)::value;
        const WsHead wh = ws_head<BYSIDE>(a, kvh * a.group + h);
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < kSlots; ++j) mx = fmaxf(mx, m_reg[j]);
        mx = wave_max(mx);
        float den = 0.0f;
#pragma unroll
        for (int j = 0; j < kSlots; ++j) {
            const int sp = lane + 64 * j;
            if (sp < SA) {
                const float f = (m_reg[j] == -INFINITY) ? 0.0f : fast_exp2(m_reg[j] - mx);
                s_w[h * kMaxSplits + sp] = f;
                den += l_reg[j] * f;
                if (sp != split) {
                    unsigned long long* rec = a.records + (int64_t)ws_row<9>(wh, sp, home[j] ? 1 : 0) * 2;
                    __hip_atomic_store(rec, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(rec + 1, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
        return wave_sum(den);
    };
    auto poll_head_n = [&](int h, float& den_out, auto slots) -> bool {
        constexpr int kSlots = decltype(slots)::value;
        float m_reg[kSlots], l_reg[kSlots];
        bool home[kSlots];  // (plain layout on this path: one home)
        const bool arrived = wait_records(h, slots, m_reg, l_reg, home);
        den_out = make_weights(h, slots, m_reg, l_reg, home);
        return arrived;
    };
    auto poll_head = [&](int h, float& den_out) -> bool {
        if (SA <= 64) return poll_head_n(h, den_out, std::integral_constant<int, 1>{});
        return poll_head_n(h, den_out, std::integral_constant<int, kMaxSplits / 64>{});
    };
    const __amdgpu_buffer_rsrc_t ws_rsrc = part_rsrc;
    constexpr int kCoherent = kCacheDevice;

    if (G <= NW || a.group <= NW) {  // (G, the group rounded up, decides it at compile time where it can)
        // One wavefront per head, all the way: poll, then read the head's partials back and write
        // its 128 outputs, without a workgroup barrier (a wave whose records are in need not wait
        // for the others). Lane = (16-byte column, half of the splits); the two halves are added
        // with one lane swap. The partials of the other workgroups were acknowledged before
        // their records were written; they are read with device-coherent 16-byte loads, a
        // lane's loads all in flight at once.
        if (spread ? wave != 0 : wave >= a.group) return;
        const int h = spread ? merge_head : wave;
        const int c4 = lane & 31;
        const int part = lane >> 5;
        const int hq = kvh * a.group + h;
        const float* w = s_w + h * kMaxSplits;
        const WsHead wh = ws_head<BYSIDE>(a, hq);
        // Byte offset of split sp's partial row, in both layouts with the same few instructions: plain, it is
        // B = row * 512; by side, the row's pair of 8 KiB blocks starts at twice B's block start and the home adds 8 KiB
        // or not: B + (B & block_mask) + home, with block_mask = 0 and home = 0 in the plain layout.
        const uint32_t row0_bytes = (uint32_t)wh.rbase * (kHeadDim * 4u);
        const uint32_t block_mask = BYSIDE ? ~(uint32_t)(kSideBlockBytes - 1) : 0u;
        const uint32_t lane_bytes = (uint32_t)c4 * 16u;
        auto load_partial = [&](int sp, uint32_t home_bytes) {
            const int spc = min(sp, SA - 1);  // in range; the weight drops the repeat
            const uint32_t B = row0_bytes + (uint32_t)spc * (kHeadDim * 4u);
            return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(ws_rsrc, B + (B & block_mask) + home_bytes + lane_bytes, 0, kCoherent));
        };
        // The first batch of partials is requested as soon as the records are in and travels
        // while the weights are worked out (they need the maximum over all records first).
        auto run = [&](auto slots, auto batch) {
            constexpr int kSlots = decltype(slots)::value;
            constexpr int kBatch = decltype(batch)::value;
            float m_reg[kSlots], l_reg[kSlots];
            bool home[kSlots];
            const bool arrived = wait_records(h, slots, m_reg, l_reg, home);
            // Which home each split's partial outputs are in: this side's, for all of them, when the workgroups of the KV
            // head share an XCD -- one constant. Otherwise (wave-uniform test) per split, from the polling lanes' flags.
            bool other = false;
#pragma unroll
            for (int j = 0; j < kSlots; ++j) other = other || home[j] != (my_xs != 0);
            const bool mixed = BYSIDE && __any(other);
            const uint32_t near_bytes = BYSIDE ? (uint32_t)(wh.ppar ^ my_xs) * kSideBlockBytes : 0u;
            float den = 0.0f;
            // The read-back, once for the usual case (every split in this side's home: one constant, nothing between the
            // loads) and once for the other one: two copies of the code rather than a test in front of every load.
            auto gather = [&](auto mixed_tag) -> f32x4 {
                auto home_bytes = [&](int sp) -> uint32_t {
                    if constexpr (!decltype(mixed_tag)::value) return near_bytes;
                    // (the flag of split spc sits in lane spc % 64, slot spc / 64 of the polling layout: the slot's flags
                    // as a 64-bit lane mask, bit spc % 64 of it -- no shuffle, and no indexed array, which the compiler
                    // would put into scratch memory)
                    const int spc = min(sp, SA - 1);
                    int xs = 0;
#pragma unroll
                    for (int j = 0; j < kSlots; ++j) {
                        const unsigned long long flags = __ballot(home[j]);
                        const int f = (int)((flags >> (spc & 63)) & 1ull);
                        xs = (spc >> 6) == j ? f : xs;
                    }
                    return (uint32_t)(wh.ppar ^ xs) * kSideBlockBytes;
                };
                f32x4 v[kBatch];
#pragma unroll
                for (int j = 0; j < kBatch; ++j) v[j] = load_partial(part + 2 * j, home_bytes(part + 2 * j));
                den = make_weights(h, slots, m_reg, l_reg, home);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wave's own weights are in LDS
                __builtin_amdgcn_wave_barrier();
                f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int j = 0; j < kBatch; ++j) {
                    const int sp = part + 2 * j;
                    sum += v[j] * (sp < SA ? w[sp] : 0.0f);
                }
                for (int s0 = part + 2 * kBatch; s0 < SA; s0 += kBatch * 2) {
#pragma unroll
                    for (int j = 0; j < kBatch; ++j) v[j] = load_partial(s0 + 2 * j, home_bytes(s0 + 2 * j));
#pragma unroll
                    for (int j = 0; j < kBatch; ++j) {
                        const int sp = s0 + 2 * j;
                        sum += v[j] * (sp < SA ? w[sp] : 0.0f);
                    }
                }
                return sum;
            };
            f32x4 acc;
            if constexpr (BYSIDE) acc = __builtin_expect(mixed, 0) ? gather(std::true_type{}) : gather(std::false_type{});
            else acc = gather(std::false_type{});
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = halves_sum(acc[e]);
            if (part == 0) {
                // A wait that ran out of patience poisons the output rather than returning a partial sum.
                const float inv = arrived ? 1.0f / den : __builtin_nanf("");
                const f32x4 r = acc * inv;
                const unsigned long long packed = (unsigned long long)pack_bf16(r[0], r[1]) | ((unsigned long long)pack_bf16(r[2], r[3]) << 32);
                unsigned long long* op = reinterpret_cast<unsigned long long*>(a.out + (int64_t)hq * kHeadDim + c4 * 4);
                if constexpr (OPROJ) __hip_atomic_store(op, packed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // read by other workgroups in this launch
                else *op = packed;
                if (a.out_f32) {
                    float* of = a.out_f32 + (int64_t)hq * kHeadDim + c4 * 4;  // only 4-byte alignment is promised
#pragma unroll
                    for (int e = 0; e < 4; ++e) of[e] = r[e];
                }
            }
            if constexpr (OPROJ) {
                // The head's output is acknowledged: say so, with the generation this launch will end on.
                // (Every workgroup of the grid read the same generation word: it moves only after all
                // heads are done.) The workers wait for all heads' tags; one wavefront of the grid (head 0
                // of the last KV head, whose workgroup is dispatched last) does too and then moves the
                // word for the next launch -- also when its wait gives up, so that tags left behind by
                // this launch can never match the next one.
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                uint32_t* done = a.ready + 4;
                const uint32_t target = proj.gen_base + 1u;
                if (lane == 0) __hip_atomic_store(done + hq, target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (kvh == (int)gridDim.x - 1 && h == 0) {
                    bool all_done = false;
                    for (int spin = 0; spin < a.max_polls; ++spin) {
                        const uint32_t d0 = __hip_atomic_load(done + min(lane, a.n_q - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        const uint32_t d1 = __hip_atomic_load(done + min(lane + 64, a.n_q - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        all_done = __all(d0 == target && d1 == target);
                        if (all_done) break;
                        __builtin_amdgcn_s_sleep(8);
                    }
                    if (lane == 0) {
                        __hip_atomic_store(a.ready, target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if (!all_done) atomicAdd(&g_poll_timeouts, 1u);
                    }
                }
            }
        };
        // (the dispatcher's own split counts stay below 64: the rare cases are kept out of the way of the usual ones)
        if (__builtin_expect(SA > 64, 0)) run(std::integral_constant<int, kMaxSplits / 64>{}, std::integral_constant<int, 16>{});
        else if (SA <= 16) run(std::integral_constant<int, 1>{}, std::integral_constant<int, 8>{});
        else run(std::integral_constant<int, 1>{}, std::integral_constant<int, 16>{});
        return;
    }

    // More heads than wavefronts: the waves take the heads in turn, then the whole workgroup
    // shares the read-back.
    bool wave_ok = true;
    for (int h = wave; h < a.group; h += NW) {
        float den;
        wave_ok = poll_head(h, den) && wave_ok;
        if (lane == 0) s_den[h] = den;
    }
    if (lane == 0) s_ok[wave] = wave_ok ? 1 : 0;
    __syncthreads();
    bool all_arrived = true;
#pragma unroll
    for (int w = 0; w < NW; ++w) all_arrived = all_arrived && s_ok[w] != 0;

    // Weighted sum of the partial outputs. Every other workgroup's partials were
    // acknowledged before its records were written; they are read with device-coherent
    // (L2-bypassing) 16-byte loads, a thread's loads all in flight at once, so that
    // the time does not depend on how the split count divides. A thread owns four
    // output columns of one head for every P-th split; the P partitions are added up
    // through LDS.
    constexpr int NT = NW * 64;
    const int units = a.group * (kHeadDim / 4);
    const int parts = units <= NT ? NT / units : 1;
    for (int u0 = 0; u0 < units; u0 += NT) {
        const int t = u0 + (int)threadIdx.x;
        const int u = t % units;
        const int part = units <= NT ? (int)threadIdx.x / units : 0;
        const bool active = (units <= NT) ? part < parts : t < units;
        const int h = u >> 5;
        const int c4 = u & 31;
        const int hq = kvh * a.group + h;
        const uint32_t base = (uint32_t)(((int64_t)hq * S * kHeadDim + c4 * 4) * (int64_t)sizeof(float));
        const float* w = s_w + h * kMaxSplits;
        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
        // All of a batch's loads are issued before the first one is used; a short list
        // of splits takes the small batch so that it does not pay for repeats.
        auto gather = [&](auto batch) {
            constexpr int kBatch = decltype(batch)::value;
            for (int s0 = part; s0 < SA; s0 += kBatch * parts) {
                f32x4 v[kBatch];
                float wv[kBatch];
#pragma unroll
                for (int j = 0; j < kBatch; ++j) {
                    const int sp = s0 + j * parts;
                    const int spc = min(sp, SA - 1);  // in range; the weight below drops the repeat
                    v[j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                                         ws_rsrc, base + (uint32_t)spc * (kHeadDim * 4u), 0, kCoherent));
                    wv[j] = sp < SA ? w[sp] : 0.0f;
                }
#pragma unroll
                for (int j = 0; j < kBatch; ++j) acc += v[j] * wv[j];
            }
        };
        if (active) {
            if (SA <= 8 * parts) gather(std::integral_constant<int, 8>{});
            else gather(std::integral_constant<int, 16>{});
        }
        if (units <= NT && parts > 1) {
            s_part[threadIdx.x] = acc;
            __syncthreads();
            if (part == 0)
                for (int pp = 1; pp < parts; ++pp) acc += s_part[pp * units + u];
        }
        if (active && part == 0) {
            // A wait that ran out of patience poisons the output rather than returning a partial sum.
            const float inv = all_arrived ? 1.0f / s_den[h] : __builtin_nanf("");
            const f32x4 r = acc * inv;
            uint16_t* op = a.out + (int64_t)hq * kHeadDim + c4 * 4;
            *reinterpret_cast<uint2*>(op) = make_uint2(pack_bf16(r[0], r[1]), pack_bf16(r[2], r[3]));
            if (a.out_f32) {
                float* of = a.out_f32 + (int64_t)hq * kHeadDim + c4 * 4;  // only 4-byte alignment is promised
#pragma unroll
                for (int e = 0; e < 4; ++e) of[e] = r[e];
            }
        }
    }
}

template <int G, int NW, int NSTAGE, bool APPEND, bool DYN, bool STAGGER = false, bool BYSIDE = false>
__global__ __launch_bounds__(NW * 64, (kWavesPerEu<G, NW>)) void mha_decode_kernel(KernelArgs a) {
    OprojState unused;
    mha_decode_body<G, NW, NSTAGE, APPEND, DYN, STAGGER, false, BYSIDE>(a, unused);
}

// The attention launch with the layer's output projection and residual add behind it, in the same launch
// (role of the pair mha_kernel_cu + fused_gemv_add_kernel_cu, code/source/model/qwen3_fused.cpp:548-552).
// A workgroup that has handed its partial results over (every one but the combiners) is idle while the
// combine runs: it requests its share of the projection's weight rows -- they do not depend on the
// attention -- and holds them in registers, waits (bounded) for every head's tag of this launch, reads the
// attention output (ordinary loads: see below) and finishes its rows: dot products, residual add, one
// rounding. The weights stream while HBM would otherwise sit idle behind the attention's hand-over.
// Needs every workgroup of the grid resident at once (the launcher checks the grid against the CU count).
template <int G, int NW, int NSTAGE, bool BYSIDE>
__global__ __launch_bounds__(NW * 64, (kWavesPerEu<G, NW>)) void mha_oproj_kernel(KernelArgs a) {
    OprojState proj;
    mha_decode_body<G, NW, NSTAGE, true, false, false, true, BYSIDE>(a, proj);
    if (!proj.worker) return;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_kv = gridDim.x;
    // Rows are dealt to the wavefronts of the workers in turn: wavefront w takes rows w, w + W, w + 2W.
    const int n_waves = n_kv * ((int)gridDim.y - 1) * NW;
    const int gw = ((int)blockIdx.y * n_kv + (int)blockIdx.x) * NW + wave;
    constexpr int kRows = kOprojRows, kSteps = kOprojSteps;
    const int k16 = a.n_q * (kHeadDim / 8);  // 16-byte chunks per weight row
    const int steps = k16 >> 6;
    const u32x4* w4 = reinterpret_cast<const u32x4*>(a.o_w);
    u32x4 wv[kRows][kSteps];
    int row[kRows];
#pragma unroll
    for (int i = 0; i < kRows; ++i) {
        row[i] = gw + i * n_waves;
        const u32x4* wr = w4 + (int64_t)min(row[i], a.o_n - 1) * k16 + lane;  // rows past the end repeat the last one and are not written
        if (i < LLMI_OPROJ_PREFETCH_ROWS) {
#pragma unroll
            for (int t = 0; t < kSteps; ++t)
                if (t < steps) wv[i][t] = __builtin_nontemporal_load(wr + t * 64);
        }
    }
    // (the residual values these rows are added to travel with the weights)
    float res_in[kRows];
#pragma unroll
    for (int i = 0; i < kRows; ++i) res_in[i] = bf16_lo((uint32_t)a.o_res[min(row[i], a.o_n - 1)]);
    // Bounded wait for the attention output: every head carries this launch's tag. One wavefront per
    // workgroup polls (a thousand wavefronts polling one line slow everything that shares its channel).
    __shared__ int s_seen;
    if (wave == 0) {
        const uint32_t* done = a.ready + 4;
        const uint32_t target = proj.gen_base + 1u;
        bool seen = false;
        for (int spin = 0; spin < a.max_polls; ++spin) {
            const uint32_t d0 = __hip_atomic_load(done + min(lane, a.n_q - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t d1 = __hip_atomic_load(done + min(lane + 64, a.n_q - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            seen = __all(d0 == target && d1 == target);
            if (seen) break;
            __builtin_amdgcn_s_sleep(4);
        }
        if (lane == 0) {
            s_seen = seen ? 1 : 0;
            if (!seen) atomicAdd(&g_poll_timeouts, 1u);
        }
    }
    __syncthreads();
    const bool ok = s_seen != 0;
    // (rows beyond the prefetch depth are fetched now)
#pragma unroll
    for (int i = LLMI_OPROJ_PREFETCH_ROWS; i < kRows; ++i) {
        const u32x4* wr = w4 + (int64_t)min(row[i], a.o_n - 1) * k16 + lane;
#pragma unroll
        for (int t = 0; t < kSteps; ++t)
            if (t < steps) wv[i][t] = __builtin_nontemporal_load(wr + t * 64);
    }
    // The attention output was written through to memory before the word moved, and no cache on this
    // side can hold an older copy: nothing in this launch has read it before, and caches do not keep
    // lines across launches. Ordinary loads, so that an XCD's L2 fetches the 8 KiB once for all its
    // workgroups (a thousand device-coherent reads of the same lines would queue at one memory channel).
    const u32x4* x4 = reinterpret_cast<const u32x4*>(a.out);
    u32x4 xv[kSteps];
#pragma unroll
    for (int t = 0; t < kSteps; ++t)
        if (t < steps) xv[t] = x4[t * 64 + lane];
#pragma unroll
    for (int i = 0; i < kRows; ++i) {
        float acc = 0.0f;
#pragma unroll
        for (int t = 0; t < kSteps; ++t)
            if (t < steps) acc = dot8_bf16(xv[t], wv[i][t], acc);
        acc = wave_sum(acc);
        // fp32 + fp32 -> bf16 once, like fused_gemv_add (matmul_kernel.cu:169-170). A wait that gave up leaves the row
        // as it was: the residual stream is updated in place, and a NaN stored there would destroy the layer's input
        // for good (the give-up is counted, and the combine's own give-up poisons the attention output).
        if (lane == 0 && row[i] < a.o_n && ok) a.o_res[row[i]] = f32_to_bf16(acc + res_in[i]);
    }
}

#ifndef LLMI_STAGES
#define LLMI_STAGES 2
#endif
#ifndef LLMI_RING_LIMIT
#define LLMI_RING_LIMIT 65536
#endif

// The layout by package side has instantiations for the wave counts the dispatcher picks itself; the planner asks
// for it nowhere else (by_side_variant).
template <int G, int NW>
constexpr bool kHasBySide = by_side_variant(G, NW);

template <int G, int NW>
void launch_decode(const KernelArgs& ka, int n_kv, bool append, hipStream_t stream) {
    // NW * NSTAGE * 8 KiB of ring must fit the LDS budget of one workgroup.
    constexpr int kStages = (NW * LLMI_STAGES * 8192 <= LLMI_RING_LIMIT) ? LLMI_STAGES : LLMI_RING_LIMIT / (NW * 8192);
    dim3 grid(n_kv, ka.num_splits);
    const bool dyn = ka.pos_dev != nullptr;  // position read at run time: its own instantiation, the static one pays nothing
    if constexpr (kHasBySide<G, NW>) {
        if (ka.by_side) {
            if (append) {
                if (dyn && ka.stagger)
                    hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, true, true, true, true>), grid, dim3(NW * 64), 0, stream, ka);
                else if (dyn) hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, true, true, false, true>), grid, dim3(NW * 64), 0, stream, ka);
                else if (ka.stagger)
                    hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, true, false, true, true>), grid, dim3(NW * 64), 0, stream, ka);
                else hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, true, false, false, true>), grid, dim3(NW * 64), 0, stream, ka);
            } else {
                if (dyn && ka.stagger)
                    hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, false, true, true, true>), grid, dim3(NW * 64), 0, stream, ka);
                else if (dyn) hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, false, true, false, true>), grid, dim3(NW * 64), 0, stream, ka);
                else if (ka.stagger)
                    hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, false, false, true, true>), grid, dim3(NW * 64), 0, stream, ka);
                else hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, false, false, false, true>), grid, dim3(NW * 64), 0, stream, ka);
            }
            return;
        }
    }
    if (append) {
        if (dyn && ka.stagger && ka.num_splits > 1)
            hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, true, true, true>), grid, dim3(NW * 64), 0, stream, ka);
        else if (dyn) hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, true, true>), grid, dim3(NW * 64), 0, stream, ka);
        else if (ka.stagger && ka.num_splits > 1)
            hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, true, false, true>), grid, dim3(NW * 64), 0, stream, ka);
        else hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, true, false>), grid, dim3(NW * 64), 0, stream, ka);
    } else {
        if (dyn && ka.stagger && ka.num_splits > 1)
            hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, false, true, true>), grid, dim3(NW * 64), 0, stream, ka);
        else if (dyn) hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, false, true>), grid, dim3(NW * 64), 0, stream, ka);
        else if (ka.stagger && ka.num_splits > 1)
            hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, false, false, true>), grid, dim3(NW * 64), 0, stream, ka);
        else hipLaunchKernelGGL((mha_decode_kernel<G, NW, kStages, false, false>), grid, dim3(NW * 64), 0, stream, ka);
    }
}

template <int G>
bool launch_decode_nw(const KernelArgs& ka, int n_kv, int nw, bool append, hipStream_t stream) {
    switch (nw) {
        case 1: launch_decode<G, 1>(ka, n_kv, append, stream); return true;
        case 2: launch_decode<G, 2>(ka, n_kv, append, stream); return true;
        case 4: launch_decode<G, 4>(ka, n_kv, append, stream); return true;
        case 8:
            if constexpr (G <= 8) { launch_decode<G, 8>(ka, n_kv, append, stream); return true; }
            return false;
        default: return false;
    }
}

template <int G, int NW>
void launch_oproj(const KernelArgs& ka, int n_kv, hipStream_t stream) {
    constexpr int kStages = (NW * LLMI_STAGES * 8192 <= LLMI_RING_LIMIT) ? LLMI_STAGES : LLMI_RING_LIMIT / (NW * 8192);
    if constexpr (kHasBySide<G, NW>) {
        if (ka.by_side) {
            hipLaunchKernelGGL((mha_oproj_kernel<G, NW, kStages, true>), dim3(n_kv, ka.num_splits), dim3(NW * 64), 0, stream, ka);
            return;
        }
    }
    hipLaunchKernelGGL((mha_oproj_kernel<G, NW, kStages, false>), dim3(n_kv, ka.num_splits), dim3(NW * 64), 0, stream, ka);
}

}  // namespace

// ---- what this translation unit exports: the launchers of its group size ----
#ifndef LLMI_GROUP
#error "define LLMI_GROUP (1, 2, 4, 8 or 16) before including mha_decode_kernels.h"
#endif
#define LLMI_CAT2(a, b) a##b
#define LLMI_CAT(a, b) LLMI_CAT2(a, b)

bool LLMI_CAT(launch_decode_group, LLMI_GROUP)(const KernelArgs& ka, int n_kv, int nw, bool append, hipStream_t stream) {
    return launch_decode_nw<LLMI_GROUP>(ka, n_kv, nw, append, stream);
}

#if LLMI_GROUP <= 8
bool LLMI_CAT(launch_oproj_group, LLMI_GROUP)(const KernelArgs& ka, int n_kv, int nw, hipStream_t stream) {
    constexpr int kWaves = LLMI_GROUP == 8 ? 8 : 4;
    if (nw != kWaves) return false;
    launch_oproj<LLMI_GROUP, kWaves>(ka, n_kv, stream);
    return true;
}
#endif

hipError_t LLMI_CAT(poll_timeouts_group, LLMI_GROUP)(unsigned int* n) {
    return hipMemcpyFromSymbol(n, HIP_SYMBOL(g_poll_timeouts), sizeof(*n));
}

}  // namespace llmi

#endif
