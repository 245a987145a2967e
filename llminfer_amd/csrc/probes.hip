// Measurement kernels (declared in llmi_hip_probes.h): a stream-only reader with the decode kernel's
// access pattern, a plain copy of known traffic, and the ping-pong probe that llmi_hip_mha_workspace_side
// decides on (the only one of them a product call uses, once per workspace allocation).

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "llmi_hip_probes.h"
#include "llmi_hip_testing.h"
#include "llmi_internal.h"
#include "side_decision.h"

namespace llmi {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Workgroup g reads tiles [g*T/G, (g+1)*T/G) of both arrays (T tiles of 4 KiB each); its wavefronts take
// the tiles of that run in turn, INFLIGHT tiles of each array requested before the first is consumed.
template <int NW, int INFLIGHT>
__global__ __launch_bounds__(NW * 64) void stream_read_kernel(const char* __restrict__ a, const char* __restrict__ b,
                                                              uint32_t tiles, uint32_t* sink) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t g = blockIdx.x, G = gridDim.x;
    const uint32_t run = tiles / G, longer = tiles % G;
    const uint32_t first = g * run + (g < longer ? g : longer);
    const uint32_t count = run + (g < longer ? 1u : 0u);
    const char* pa = a + (size_t)first * 4096u + lane * 16u;
    const char* pb = b + (size_t)first * 4096u + lane * 16u;
    u32x4 acc = {0u, 0u, 0u, 0u};
    for (uint32_t t0 = wave; t0 < count; t0 += NW * INFLIGHT) {
        u32x4 r[INFLIGHT][8];
#pragma unroll
        for (int u = 0; u < INFLIGHT; ++u) {
            uint32_t t = t0 + u * NW;
            if (t >= count) t = t0;  // (a repeat near the end of the run: served by the cache, never out of range)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                r[u][j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(pa + (size_t)t * 4096u + j * 1024u));
                r[u][4 + j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(pb + (size_t)t * 4096u + j * 1024u));
            }
        }
#pragma unroll
        for (int u = 0; u < INFLIGHT; ++u)
#pragma unroll
            for (int j = 0; j < 8; ++j) acc ^= r[u][j];
    }
    // Keeps the loads alive; the condition does not hold for any data a benchmark feeds it.
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u && sink) sink[0] = acc[0];
}

// The same stream in the position-major cache layout: the arrays are rows of `row_bytes` bytes, a KV head's part of a row
// is 256 bytes at offset 256 * head. Workgroup (head, g) reads its head's pieces of a contiguous run of 16-row tiles;
// a load instruction takes four rows (one per 16 lanes), like the decode kernel's.
template <int NW, int INFLIGHT>
__global__ __launch_bounds__(NW * 64) void stream_read_rows_kernel(const char* __restrict__ a, const char* __restrict__ b,
                                                                   uint32_t tiles, uint32_t row_bytes, uint32_t* sink) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t head = blockIdx.x, g = blockIdx.y, G = gridDim.y;
    const uint32_t run = tiles / G, longer = tiles % G;
    const uint32_t first = g * run + (g < longer ? g : longer);
    const uint32_t count = run + (g < longer ? 1u : 0u);
    const size_t lane_off = (size_t)(first * 16u + (lane >> 4)) * row_bytes + head * 256u + (lane & 15u) * 16u;
    const char* pa = a + lane_off;
    const char* pb = b + lane_off;
    u32x4 acc = {0u, 0u, 0u, 0u};
    for (uint32_t t0 = wave; t0 < count; t0 += NW * INFLIGHT) {
        u32x4 r[INFLIGHT][8];
#pragma unroll
        for (int u = 0; u < INFLIGHT; ++u) {
            uint32_t t = t0 + u * NW;
            if (t >= count) t = t0;  // (a repeat near the end of the run: served by the cache, never out of range)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const size_t off = (size_t)(t * 16u + 4u * j) * row_bytes;
                r[u][j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(pa + off));
                r[u][4 + j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(pb + off));
            }
        }
#pragma unroll
        for (int u = 0; u < INFLIGHT; ++u)
#pragma unroll
            for (int j = 0; j < 8; ++j) acc ^= r[u][j];
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u && sink) sink[0] = acc[0];
}

// The decode kernel's K/V stream without its arithmetic, one feature at a time: the same grid (KV head x split, the
// KV head fastest), the same deal of 16-position tiles to splits and wavefronts, NSTAGE tiles in flight per wavefront.
//   MODE 0: ordinary non-temporal loads to registers, a lane's 16 bytes at its own offset of the row (the floor kernel's way)
//   MODE 1: LDS-DMA loads (global_load_lds_dwordx4 nt) into a per-wavefront ring, whole rows per instruction
//   MODE 2: MODE 1 with the K chunks swizzled by row & 7 -- exactly what the decode kernel requests
//   MODE 3: MODE 2 with a pause of `pause` x 64 clocks after every tile has landed: a wavefront that does its
//           arithmetic is not requesting
// `rs`: bytes between consecutive positions of one KV head (256 head-major, 256 x KV heads position-major);
// `stagger`: the splits start their walks at different tiles (the decode kernel's STAGGER).
__device__ __forceinline__ void probe_dma16(const char* base, uint32_t voff, uint32_t lds_off) {
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b);
    const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
    const uint64_t sbase = ((uint64_t)b_hi << 32) | (uint64_t)b_lo;
    const uint32_t slds = (uint32_t)__builtin_amdgcn_readfirstlane(lds_off);
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt" :: "v"(voff), "s"(sbase), "{m0}"(slds) : "memory");
}

template <int NW, int NSTAGE, int MODE>
__global__ __launch_bounds__(NW * 64) void stream_tiles_kernel(const char* __restrict__ k, const char* __restrict__ v, int tiles_per_head,
                                                               int64_t head_bytes, uint32_t rs, int pause, int stagger, uint32_t* sink) {
    __shared__ __attribute__((aligned(1024))) char smem[MODE == 0 ? 1024 : NW * NSTAGE * 8192];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n16 = lane & 15, kg = lane >> 4;
    // (stagger bit 1: the grid has the splits fastest -- consecutive workgroups read consecutive runs of one head --
    // instead of the decode kernel's KV heads fastest)
    const bool splits_fastest = (stagger & 2) != 0;
    const int rot_mask = (stagger & 1) ? 3 : (stagger >> 2);  // (bits 2 and up: another mask for the rotation)
    const int kvh = splits_fastest ? blockIdx.y : blockIdx.x, split = splits_fastest ? blockIdx.x : blockIdx.y;
    const int S = splits_fastest ? gridDim.x : gridDim.y;
    const int run = tiles_per_head / S, longer = tiles_per_head % S;
    const int ntiles = run + (split < longer ? 1 : 0);
    const int begin = split * run + min(split, longer);
    const char* kb = k + kvh * head_bytes + (int64_t)begin * 16 * rs;
    const char* vb = v + kvh * head_bytes + (int64_t)begin * 16 * rs;
    const int n_my = wave < ntiles ? (ntiles - wave + NW - 1) / NW : 0;
    const int rot = min(split & rot_mask, max(n_my - 1, 0));
    auto tile_of = [&](int i) {
        int ii = i + rot;
        if (ii >= n_my) ii -= n_my;
        return wave + ii * NW;
    };
    const uint32_t k_row = kg * rs, col_lin = n16 * 16u;
    const uint32_t k_col0 = MODE >= 2 ? (uint32_t)(n16 ^ kg) * 16u : col_lin;
    const uint32_t k_col1 = MODE >= 2 ? (uint32_t)(n16 ^ (4 + kg)) * 16u : col_lin;
    u32x4 acc = {0u, 0u, 0u, 0u};
    if constexpr (MODE == 0) {
        for (int i0 = 0; i0 < n_my; i0 += NSTAGE) {
            u32x4 r[NSTAGE][8];
#pragma unroll
            for (int u = 0; u < NSTAGE; ++u) {
                const uint32_t base = (uint32_t)tile_of(min(i0 + u, n_my - 1)) * 16u * rs + k_row + col_lin;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    r[u][j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kb + base + j * 4 * rs));
                    r[u][4 + j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vb + base + j * 4 * rs));
                }
            }
#pragma unroll
            for (int u = 0; u < NSTAGE; ++u)
#pragma unroll
                for (int j = 0; j < 8; ++j) acc ^= r[u][j];
        }
    } else {
        const uint32_t ring = (uint32_t)(uintptr_t)(smem + wave * NSTAGE * 8192);
        auto issue = [&](int i, int stage) {
            const uint32_t base = (uint32_t)tile_of(i) * 16u * rs;
            const uint32_t slot = ring + stage * 8192u;
#pragma unroll
            for (int j = 0; j < 4; ++j) probe_dma16(kb, base + k_row + j * 4u * rs + ((j & 1) ? k_col1 : k_col0), slot + j * 1024);
#pragma unroll
            for (int j = 0; j < 4; ++j) probe_dma16(vb, base + k_row + j * 4u * rs + col_lin, slot + 4096 + j * 1024);
        };
        for (int s0 = 0; s0 < NSTAGE; ++s0)
            if (s0 < n_my) issue(s0, s0);
        int stage = 0;
        for (int i = 0; i < n_my; ++i) {
            const int newer = min(NSTAGE - 1, n_my - 1 - i);
            if (newer <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            else if (newer == 1) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            else if (newer == 2) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
            acc ^= *reinterpret_cast<const u32x4*>(smem + wave * NSTAGE * 8192 + stage * 8192 + lane * 16);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (i + NSTAGE < n_my) issue(i + NSTAGE, stage);
            if constexpr (MODE == 3)
                for (int p = 0; p < pause; ++p) __builtin_amdgcn_s_sleep(1);
            stage = (stage + 1 == NSTAGE) ? 0 : stage + 1;
        }
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u && sink) sink[0] = acc[0];
}

__global__ __launch_bounds__(256) void copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

__device__ __forceinline__ uint32_t xcc_id() {
    uint32_t x;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
    return x & 15u;
}

// Device-scope (sc1) 4-byte load and store, each waited for: what the fused combine's hand-over uses.
__device__ __forceinline__ uint32_t load_device_scope(const uint32_t* p) {
    uint32_t v;
    asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ void store_device_scope(uint32_t* p, uint32_t v) {
    asm volatile("global_store_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" ::"v"(p), "v"(v) : "memory");
}

// Hand-over latency from every XCD through two blocks of memory. Workgroups i and i + 8 of a grid of 16 (one XCD when
// workgroups are dealt to the XCDs in turn) play ping-pong through two words of their own 256-byte line in block `a`,
// then in block `b`, twice each: i stores a number (device scope), i + 8 polls for it and stores it into the second
// word, i polls for that. kPingPongs round trips per chain; every poll loop is bounded, a pair that loses a number
// gives up and says so. Workgroup i < 8 reports: its XCD, its partner's, the ticks (10 ns) spent on a and on b, 1 if
// every number arrived.
constexpr int kPingPongPolls = 4000;  // (kPingPongs round trips per chain, kPingPongChains chains: side_decision.h)
__global__ __launch_bounds__(64) void block_pingpong_kernel(uint32_t* a, uint32_t* b, uint32_t* out) {
    if (threadIdx.x != 0) return;
    const int pair = blockIdx.x & 7;
    const bool leader = blockIdx.x < 8;
    uint32_t* xcc_partner = out + 8 * pair + 5;  // (written by the partner, plainly: read by the host only)
    if (!leader) *xcc_partner = xcc_id();
    unsigned long long t[2] = {0, 0};
    uint32_t ok = 1, seq = 0;
    for (int c = 0; c < kPingPongChains && ok; ++c)
        for (int which = 0; which < 2 && ok; ++which) {
            uint32_t* line = (which ? b : a) + pair * 64;  // this pair's 256 bytes of the block
            uint32_t* ping = line;
            uint32_t* pong = line + 16;
            const unsigned long long t0 = wall_clock64();
            for (int i = 0; i < kPingPongs && ok; ++i) {
                ++seq;
                uint32_t* mine = leader ? ping : pong;
                const uint32_t* theirs = leader ? pong : ping;
                if (leader) store_device_scope(mine, seq);
                int polls = 0;
                while (polls < kPingPongPolls && load_device_scope(theirs) != seq) ++polls;
                if (polls == kPingPongPolls) ok = 0;
                if (!leader) store_device_scope(mine, seq);
            }
            t[which] += wall_clock64() - t0;
        }
    if (leader) {
        out[8 * pair + 0] = xcc_id();
        out[8 * pair + 1] = (uint32_t)t[0];
        out[8 * pair + 2] = (uint32_t)t[1];
        out[8 * pair + 3] = ok;
    }
}

template <int NW>
bool launch_stream(int inflight, dim3 grid, hipStream_t s, const char* a, const char* b, uint32_t tiles, uint32_t* sink) {
    switch (inflight) {
        case 1: hipLaunchKernelGGL((stream_read_kernel<NW, 1>), grid, dim3(NW * 64), 0, s, a, b, tiles, sink); return true;
        case 2: hipLaunchKernelGGL((stream_read_kernel<NW, 2>), grid, dim3(NW * 64), 0, s, a, b, tiles, sink); return true;
        case 4: hipLaunchKernelGGL((stream_read_kernel<NW, 4>), grid, dim3(NW * 64), 0, s, a, b, tiles, sink); return true;
        default: return false;
    }
}

template <int NW, int NSTAGE>
bool launch_stream_tiles(int mode, dim3 grid, hipStream_t s, const char* k, const char* v, int tiles, int64_t head_bytes, uint32_t rs,
                         int pause, int stagger, uint32_t* sink) {
    const dim3 block(NW * 64);
    switch (mode) {
        case 0: hipLaunchKernelGGL((stream_tiles_kernel<NW, NSTAGE, 0>), grid, block, 0, s, k, v, tiles, head_bytes, rs, pause, stagger, sink); return true;
        case 1: hipLaunchKernelGGL((stream_tiles_kernel<NW, NSTAGE, 1>), grid, block, 0, s, k, v, tiles, head_bytes, rs, pause, stagger, sink); return true;
        case 2: hipLaunchKernelGGL((stream_tiles_kernel<NW, NSTAGE, 2>), grid, block, 0, s, k, v, tiles, head_bytes, rs, pause, stagger, sink); return true;
        case 3: hipLaunchKernelGGL((stream_tiles_kernel<NW, NSTAGE, 3>), grid, block, 0, s, k, v, tiles, head_bytes, rs, pause, stagger, sink); return true;
        default: return false;
    }
}

template <int NW>
bool launch_stream_rows(int inflight, dim3 grid, hipStream_t s, const char* a, const char* b, uint32_t tiles, uint32_t row_bytes,
                        uint32_t* sink) {
    switch (inflight) {
        case 1: hipLaunchKernelGGL((stream_read_rows_kernel<NW, 1>), grid, dim3(NW * 64), 0, s, a, b, tiles, row_bytes, sink); return true;
        case 2: hipLaunchKernelGGL((stream_read_rows_kernel<NW, 2>), grid, dim3(NW * 64), 0, s, a, b, tiles, row_bytes, sink); return true;
        case 4: hipLaunchKernelGGL((stream_read_rows_kernel<NW, 4>), grid, dim3(NW * 64), 0, s, a, b, tiles, row_bytes, sink); return true;
        default: return false;
    }
}

}  // namespace
}  // namespace llmi

namespace llmi {

// Which 8 KiB blocks lie near which side of the package, seen from the workspace itself: the time of hand-overs between
// two workgroups of one XCD (block_pingpong_kernel, all eight XCDs at once, each pair reporting the XCD it ran on)
// through a block with address bit 13 clear and through its neighbour with the bit set. One run gives one decision
// (side_from_pingpong: the two sides of the package must disagree about which block is nearer, each clearly); the
// answer is a side only when two runs name it and none names the other (side_agreement), else "no statement" (0).
// What it answered is counted (llmi_hip_workspace_side_stats).
static std::atomic<unsigned long long> g_side_stats[3];
static int measure_window_side(char* window, hipStream_t stream, int* side) {
    *side = 0;
    // The pairs' lines: the first 2 KiB of either block; the results: the second 4 KiB of the first block.
    uint32_t* out = reinterpret_cast<uint32_t*>(window + 4096);
    constexpr int kRuns = 4;
    int decisions[kRuns];
    int runs = 0, verdict = kSideAbstained;
    while (runs < kRuns) {
        if (int rc = llmi_hip_probe_block_pingpong(window, window + kSideBlock, out, stream)) return rc;
        uint32_t r[64];
        if (int rc = record_hip_error(hipMemcpyAsync(r, out, sizeof(r), hipMemcpyDeviceToHost, stream), "hipMemcpyAsync")) return rc;
        if (int rc = record_hip_error(hipStreamSynchronize(stream), "hipStreamSynchronize")) return rc;
        decisions[runs++] = side_from_pingpong(r);
        *side = side_agreement(decisions, runs, &verdict);
        if (verdict != kSideAbstained) break;  // two runs agree, or two contradict each other: more runs change neither
    }
    g_side_stats[verdict].fetch_add(1, std::memory_order_relaxed);
    return LLMI_OK;
}

// One window per 2 MiB-aligned region the workspace reaches into: the first 16 KiB-aligned 16 KiB of the region that
// lie inside the workspace.
int measure_workspace_side(void* workspace, size_t bytes, hipStream_t stream, int32_t* sides) {
    *sides = 0;
    const uintptr_t w0 = reinterpret_cast<uintptr_t>(workspace), w1 = w0 + bytes;
    uint32_t word = 0;
    bool any = false;
    for (uintptr_t i = 0; i < 16; ++i) {
        const uintptr_t region = ((w0 >> 21) + i) << 21;
        if (region >= w1) break;
        uintptr_t window = region > w0 ? region : w0;
        window = (window + 2 * kSideBlock - 1) & ~(uintptr_t)(2 * kSideBlock - 1);
        if (window + 2 * kSideBlock > w1 || window + 2 * kSideBlock > region + (1u << 21)) continue;
        int side = 0;
        if (int rc = measure_window_side(reinterpret_cast<char*>(window), stream, &side)) return rc;
        word |= (uint32_t)side << (2 * i);
        any = true;
    }
    if (!any) return LLMI_ERR_WORKSPACE;
    *sides = (int32_t)word;
    return LLMI_OK;
}

}  // namespace llmi

using namespace llmi;

extern "C" {

int llmi_hip_probe_stream_read(const void* a, const void* b, size_t bytes_each, int32_t workgroups, int32_t waves,
                               int32_t tiles_in_flight, void* sink, void* stream) {
    if (!a || !b || !sink) return LLMI_ERR_NULL_POINTER;
    if (bytes_each == 0 || bytes_each % 4096 != 0 || bytes_each / 4096 > 0xffffffffull) return LLMI_ERR_INVALID_ARG;
    if (workgroups < 1 || workgroups > 65535) return LLMI_ERR_INVALID_ARG;
    if (((uintptr_t)a | (uintptr_t)b) & 15u) return LLMI_ERR_ALIGNMENT;
    const uint32_t tiles = (uint32_t)(bytes_each / 4096);
    const char* pa = static_cast<const char*>(a);
    const char* pb = static_cast<const char*>(b);
    uint32_t* ps = static_cast<uint32_t*>(sink);
    hipStream_t s = static_cast<hipStream_t>(stream);
    bool ok = false;
    switch (waves) {
        case 1: ok = launch_stream<1>(tiles_in_flight, dim3(workgroups), s, pa, pb, tiles, ps); break;
        case 2: ok = launch_stream<2>(tiles_in_flight, dim3(workgroups), s, pa, pb, tiles, ps); break;
        case 4: ok = launch_stream<4>(tiles_in_flight, dim3(workgroups), s, pa, pb, tiles, ps); break;
        case 8: ok = launch_stream<8>(tiles_in_flight, dim3(workgroups), s, pa, pb, tiles, ps); break;
        default: ok = false;
    }
    if (!ok) return LLMI_ERR_INVALID_ARG;
    return check_launch();
}

int llmi_hip_probe_stream_read_rows(const void* a, const void* b, int32_t rows, int32_t heads, int32_t workgroups_per_head,
                                    int32_t waves, int32_t tiles_in_flight, void* sink, void* stream) {
    if (!a || !b || !sink) return LLMI_ERR_NULL_POINTER;
    if (rows < 16 || rows % 16 != 0 || heads < 1 || heads > 256) return LLMI_ERR_INVALID_ARG;
    if (workgroups_per_head < 1 || workgroups_per_head > 65535 || workgroups_per_head > rows / 16) return LLMI_ERR_INVALID_ARG;
    if (((uintptr_t)a | (uintptr_t)b) & 15u) return LLMI_ERR_ALIGNMENT;
    const uint32_t tiles = (uint32_t)(rows / 16);
    const uint32_t row_bytes = (uint32_t)heads * 256u;
    const char* pa = static_cast<const char*>(a);
    const char* pb = static_cast<const char*>(b);
    uint32_t* ps = static_cast<uint32_t*>(sink);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)heads, (unsigned)workgroups_per_head);
    bool ok = false;
    switch (waves) {
        case 1: ok = launch_stream_rows<1>(tiles_in_flight, grid, s, pa, pb, tiles, row_bytes, ps); break;
        case 2: ok = launch_stream_rows<2>(tiles_in_flight, grid, s, pa, pb, tiles, row_bytes, ps); break;
        case 4: ok = launch_stream_rows<4>(tiles_in_flight, grid, s, pa, pb, tiles, row_bytes, ps); break;
        case 8: ok = launch_stream_rows<8>(tiles_in_flight, grid, s, pa, pb, tiles, row_bytes, ps); break;
        default: ok = false;
    }
    if (!ok) return LLMI_ERR_INVALID_ARG;
    return check_launch();
}

int llmi_hip_probe_stream_tiles(const void* k, const void* v, int32_t positions, int32_t kv_heads, int32_t kv_layout, int32_t splits,
                                int32_t waves, int32_t tiles_in_flight, int32_t mode, int32_t pause, int32_t stagger, void* sink, void* stream) {
    if (!k || !v || !sink) return LLMI_ERR_NULL_POINTER;
    if (positions < 16 || positions % 16 != 0 || kv_heads < 1 || kv_heads > 1024) return LLMI_ERR_INVALID_ARG;
    if (splits < 1 || splits > 65535 || splits > positions / 16) return LLMI_ERR_INVALID_ARG;
    if (kv_layout != LLMI_KV_LAYOUT_POS_MAJOR && kv_layout != LLMI_KV_LAYOUT_HEAD_MAJOR) return LLMI_ERR_LAYOUT;
    if (mode < 0 || mode > 3 || pause < 0 || pause > 1024) return LLMI_ERR_INVALID_ARG;
    if (((uintptr_t)k | (uintptr_t)v) & 15u) return LLMI_ERR_ALIGNMENT;
    const bool pm = kv_layout == LLMI_KV_LAYOUT_POS_MAJOR;
    const uint32_t rs = pm ? (uint32_t)kv_heads * 256u : 256u;
    const int64_t head_bytes = pm ? 256 : (int64_t)positions * 256;
    if ((uint64_t)positions * rs > 0xffffffffull) return LLMI_ERR_INVALID_ARG;  // (32-bit offsets inside a head's run)
    if (stagger < 0 || stagger > 255) return LLMI_ERR_INVALID_ARG;
    const dim3 grid = (stagger & 2) ? dim3((unsigned)splits, (unsigned)kv_heads) : dim3((unsigned)kv_heads, (unsigned)splits);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const char* kp = static_cast<const char*>(k);
    const char* vp = static_cast<const char*>(v);
    uint32_t* ps = static_cast<uint32_t*>(sink);
    const int tiles = positions / 16;
    bool ok = false;
    if (waves == 4 && tiles_in_flight == 2) ok = launch_stream_tiles<4, 2>(mode, grid, s, kp, vp, tiles, head_bytes, rs, pause, stagger, ps);
    else if (waves == 8 && tiles_in_flight == 1) ok = launch_stream_tiles<8, 1>(mode, grid, s, kp, vp, tiles, head_bytes, rs, pause, stagger, ps);
    else if (waves == 8 && tiles_in_flight == 2) ok = launch_stream_tiles<8, 2>(mode, grid, s, kp, vp, tiles, head_bytes, rs, pause, stagger, ps);
    else if (waves == 4 && tiles_in_flight == 4) ok = launch_stream_tiles<4, 4>(mode, grid, s, kp, vp, tiles, head_bytes, rs, pause, stagger, ps);
    if (!ok) return LLMI_ERR_INVALID_ARG;
    return check_launch();
}

int llmi_hip_probe_copy(const void* src, void* dst, size_t bytes, void* stream) {
    if (!src || !dst) return LLMI_ERR_NULL_POINTER;
    if (bytes == 0 || bytes % 16 != 0) return LLMI_ERR_INVALID_ARG;
    if (((uintptr_t)src | (uintptr_t)dst) & 15u) return LLMI_ERR_ALIGNMENT;
    hipLaunchKernelGGL(copy_kernel, dim3(2048), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), bytes / 16);
    return check_launch();
}

int llmi_hip_probe_block_pingpong(void* a, void* b, uint32_t* out, void* stream) {
    if (!a || !b || !out) return LLMI_ERR_NULL_POINTER;
    if (((uintptr_t)a | (uintptr_t)b) & 255u) return LLMI_ERR_ALIGNMENT;
    if ((uintptr_t)out & 3u) return LLMI_ERR_ALIGNMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // (numbers start at 1: the lines and the result start from zero)
    if (int rc = record_hip_error(hipMemsetAsync(a, 0, 2048, s), "hipMemsetAsync")) return rc;
    if (int rc = record_hip_error(hipMemsetAsync(b, 0, 2048, s), "hipMemsetAsync")) return rc;
    if (int rc = record_hip_error(hipMemsetAsync(out, 0, 64 * sizeof(uint32_t), s), "hipMemsetAsync")) return rc;
    hipLaunchKernelGGL(block_pingpong_kernel, dim3(16), dim3(64), 0, s, static_cast<uint32_t*>(a), static_cast<uint32_t*>(b), out);
    return check_launch();
}

int32_t llmi_hip_side_from_pingpong(const uint32_t* results64) { return results64 ? side_from_pingpong(results64) : 0; }

int32_t llmi_hip_side_agreement(const int32_t* decisions, int32_t count, int32_t* verdict) {
    if (!decisions || count < 0) {
        if (verdict) *verdict = kSideAbstained;
        return 0;
    }
    int v = kSideAbstained;
    const int side = side_agreement(decisions, count, &v);
    if (verdict) *verdict = v;
    return side;
}

void llmi_hip_workspace_side_stats(uint64_t out[3]) {
    if (!out) return;
    for (int i = 0; i < 3; ++i) out[i] = g_side_stats[i].load(std::memory_order_relaxed);
}

}  // extern "C"
