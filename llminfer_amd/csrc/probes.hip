// Measurement kernels (declared in llmi_hip_probes.h): a stream-only reader with the decode kernel's
// access pattern, a plain copy of known traffic, and a two-workgroup hand-over probe. Nothing here
// is on the product path.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "llmi_hip_probes.h"
#include "llmi_internal.h"

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

__global__ __launch_bounds__(256) void copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

__device__ __forceinline__ uint32_t xcc_id() {
    uint32_t x;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
    return x & 15u;
}

template <int M>
__device__ __forceinline__ uint32_t load_policy(const uint32_t* p) {
    uint32_t v;
    if constexpr (M == LLMI_PROBE_PLAIN) asm volatile("global_load_dword %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    if constexpr (M == LLMI_PROBE_SC0) asm volatile("global_load_dword %0, %1, off sc0\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    if constexpr (M == LLMI_PROBE_SC1) asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    if constexpr (M == LLMI_PROBE_SC0_SC1) asm volatile("global_load_dword %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    if constexpr (M == LLMI_PROBE_NT) asm volatile("global_load_dword %0, %1, off nt\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    return v;
}
template <int M>
__device__ __forceinline__ void store_policy(uint32_t* p, uint32_t v) {
    if constexpr (M == LLMI_PROBE_PLAIN) asm volatile("global_store_dword %0, %1, off\n\ts_waitcnt vmcnt(0)" ::"v"(p), "v"(v) : "memory");
    if constexpr (M == LLMI_PROBE_SC0) asm volatile("global_store_dword %0, %1, off sc0\n\ts_waitcnt vmcnt(0)" ::"v"(p), "v"(v) : "memory");
    if constexpr (M == LLMI_PROBE_SC1) asm volatile("global_store_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" ::"v"(p), "v"(v) : "memory");
    if constexpr (M == LLMI_PROBE_SC0_SC1) asm volatile("global_store_dword %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" ::"v"(p), "v"(v) : "memory");
    if constexpr (M == LLMI_PROBE_NT) asm volatile("global_store_dword %0, %1, off nt\n\ts_waitcnt vmcnt(0)" ::"v"(p), "v"(v) : "memory");
}

constexpr uint32_t kProbeValue = 42u;
constexpr uint32_t kProbePolls = 4000u;

// line[0]: the data word; line[64] (another 256-byte line): reader -> writer "I am polling".
template <int WM, int RM>
__global__ __launch_bounds__(64) void handover_kernel(uint32_t* line, llmi_probe_handover_result* res, int writer_wg, int reader_wg, int precache) {
    if (threadIdx.x != 0) return;
    uint32_t* data = line;
    uint32_t* flag = line + 64;
    if ((int)blockIdx.x == reader_wg) {
        if (precache) (void)(load_policy<LLMI_PROBE_PLAIN>(data) + load_policy<RM>(data));
        store_policy<LLMI_PROBE_SC1>(flag, 1u);
        const unsigned long long t0 = wall_clock64();
        uint32_t polls = 0, seen = 0;
        for (; polls < kProbePolls; ++polls)
            if (load_policy<RM>(data) == kProbeValue) {
                seen = 1;
                break;
            }
        const unsigned long long t1 = wall_clock64();
        res->seen = seen;
        res->polls = polls;
        res->ns = (uint32_t)((t1 - t0) * 10ull);
        res->xcc_reader = xcc_id();
    } else if ((int)blockIdx.x == writer_wg) {
        res->xcc_writer = xcc_id();
        for (int i = 0; i < 200000; ++i)  // bounded: the reader raises the flag at once
            if (load_policy<LLMI_PROBE_SC1>(flag) == 1u) break;
        const unsigned long long t0 = wall_clock64();
        while (wall_clock64() - t0 < 200ull) {  // 2 us: the reader is polling by now
        }
        store_policy<WM>(data, kProbeValue);
    }
}

// Where the workgroups of a launch land: every workgroup (256 threads, LDS bytes of LDS: the footprint of a
// decode workgroup, or more than half a CU's LDS so that two cannot share a CU) records the XCD and the
// hardware id register of the CU it runs on, then keeps its CU for hold_ticks of the 100 MHz clock (bounded),
// so that the whole grid is resident at once like the decode kernel's.
template <int LDS>
__global__ __launch_bounds__(256) void placement_kernel(uint32_t* out, uint32_t hold_ticks) {
    __shared__ char pad[LDS];
    if (threadIdx.x == 0) {
        *reinterpret_cast<volatile char*>(pad) = 1;  // (keeps the allocation)
        uint32_t hw;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw));
        out[2 * blockIdx.x] = xcc_id();
        out[2 * blockIdx.x + 1] = hw;
    }
    const unsigned long long t0 = wall_clock64();
    for (int i = 0; i < 100000; ++i) {  // bounded: 100 us at the most with the sleep below
        if (wall_clock64() - t0 >= hold_ticks) break;
        __builtin_amdgcn_s_sleep(8);
    }
}

// Hand-over latency from every XCD through two blocks of memory. Workgroups i and i + 8 of a grid of 16 (one XCD when
// workgroups are dealt to the XCDs in turn) play ping-pong through two words of their own 256-byte line in block `a`,
// then in block `b`, twice each: i stores a number (device scope), i + 8 polls for it and stores it into the second
// word, i polls for that. kPingPongs round trips per chain; every poll loop is bounded, a pair that loses a number
// gives up and says so. Workgroup i < 8 reports: its XCD, its partner's, the ticks (10 ns) spent on a and on b, 1 if
// every number arrived.
constexpr int kPingPongs = 16, kPingPongChains = 2, kPingPongPolls = 4000;
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
                if (leader) store_policy<LLMI_PROBE_SC1>(mine, seq);
                int polls = 0;
                while (polls < kPingPongPolls && load_policy<LLMI_PROBE_SC1>(theirs) != seq) ++polls;
                if (polls == kPingPongPolls) ok = 0;
                if (!leader) store_policy<LLMI_PROBE_SC1>(mine, seq);
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

typedef void (*HandoverKernel)(uint32_t*, llmi_probe_handover_result*, int, int, int);
template <int WM>
HandoverKernel pick_reader(int rm) {
    switch (rm) {
        case LLMI_PROBE_PLAIN: return handover_kernel<WM, LLMI_PROBE_PLAIN>;
        case LLMI_PROBE_SC0: return handover_kernel<WM, LLMI_PROBE_SC0>;
        case LLMI_PROBE_SC1: return handover_kernel<WM, LLMI_PROBE_SC1>;
        case LLMI_PROBE_SC0_SC1: return handover_kernel<WM, LLMI_PROBE_SC0_SC1>;
        default: return handover_kernel<WM, LLMI_PROBE_NT>;
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
// through a block with address bit 13 clear and through its neighbour with the bit set. The two sides of the package
// must disagree about which block is nearer, each clearly: anything else is reported as "no statement" (0).
static int measure_window_side(char* window, hipStream_t stream, int* side) {
    *side = 0;
    // The pairs' lines: the first 2 KiB of either block; the results: the second 4 KiB of the first block.
    uint32_t* out = reinterpret_cast<uint32_t*>(window + 4096);
    for (int attempt = 0; attempt < 3; ++attempt) {
        if (int rc = llmi_hip_probe_block_pingpong(window, window + kSideBlock, out, stream)) return rc;
        uint32_t r[8][8];
        if (int rc = record_hip_error(hipMemcpyAsync(r, out, sizeof(r), hipMemcpyDeviceToHost, stream), "hipMemcpyAsync")) return rc;
        if (int rc = record_hip_error(hipStreamSynchronize(stream), "hipStreamSynchronize")) return rc;
        long long diff[2] = {0, 0};  // per side of the package: ticks through the clear block minus ticks through the set block
        int n[2] = {0, 0};
        for (int p = 0; p < 8; ++p) {
            if (!r[p][3] || r[p][0] != r[p][5]) continue;  // a pair that lost a number, or did not share an XCD
            const int sd = (int)(r[p][0] >> 2) & 1;
            diff[sd] += (long long)r[p][1] - (long long)r[p][2];
            ++n[sd];
        }
        if (n[0] < 2 || n[1] < 2) continue;
        // Per hand-over (two per round trip), in ns (a tick is 10 ns).
        const long long handovers = 2ll * kPingPongs * kPingPongChains;
        const long long d0 = diff[0] * 10 / (n[0] * handovers), d4 = diff[1] * 10 / (n[1] * handovers);
        constexpr long long kThresholdNs = 25;
        if (d0 <= -kThresholdNs && d4 >= kThresholdNs) *side = 1;       // XCDs 0-3 are nearer to the clear block, 4-7 to the set one
        else if (d0 >= kThresholdNs && d4 <= -kThresholdNs) *side = 2;
        if (*side) break;
    }
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

int llmi_hip_probe_placement(int32_t workgroups, int32_t exclusive, uint32_t* ids, void* stream) {
    if (!ids) return LLMI_ERR_NULL_POINTER;
    if (workgroups < 1 || workgroups > 4096) return LLMI_ERR_INVALID_ARG;
    if ((uintptr_t)ids & 3u) return LLMI_ERR_ALIGNMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint32_t hold = 500;  // 5 us
    if (exclusive) hipLaunchKernelGGL((placement_kernel<84 * 1024>), dim3(workgroups), dim3(256), 0, s, ids, hold);
    else hipLaunchKernelGGL((placement_kernel<66 * 1024>), dim3(workgroups), dim3(256), 0, s, ids, hold);
    return check_launch();
}

int llmi_hip_probe_handover(int32_t store_pol, int32_t load_pol, int32_t writer_workgroup, int32_t reader_workgroup, int32_t precache, void* line,
                            llmi_probe_handover_result* result, void* stream) {
    if (!line || !result) return LLMI_ERR_NULL_POINTER;
    if (store_pol < 0 || store_pol > LLMI_PROBE_NT || load_pol < 0 || load_pol > LLMI_PROBE_NT) return LLMI_ERR_INVALID_ARG;
    if (writer_workgroup < 0 || writer_workgroup > 15 || reader_workgroup < 0 || reader_workgroup > 15 || writer_workgroup == reader_workgroup)
        return LLMI_ERR_INVALID_ARG;
    if ((uintptr_t)line & 255u) return LLMI_ERR_ALIGNMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (int rc = record_hip_error(hipMemsetAsync(line, 0, 4096, s), "hipMemsetAsync")) return rc;
    if (int rc = record_hip_error(hipMemsetAsync(result, 0, sizeof(*result), s), "hipMemsetAsync")) return rc;
    HandoverKernel k;
    switch (store_pol) {
        case LLMI_PROBE_PLAIN: k = pick_reader<LLMI_PROBE_PLAIN>(load_pol); break;
        case LLMI_PROBE_SC0: k = pick_reader<LLMI_PROBE_SC0>(load_pol); break;
        case LLMI_PROBE_SC1: k = pick_reader<LLMI_PROBE_SC1>(load_pol); break;
        case LLMI_PROBE_SC0_SC1: k = pick_reader<LLMI_PROBE_SC0_SC1>(load_pol); break;
        default: k = pick_reader<LLMI_PROBE_NT>(load_pol); break;
    }
    hipLaunchKernelGGL(k, dim3(16), dim3(64), 0, s, static_cast<uint32_t*>(line), result, (int)writer_workgroup, (int)reader_workgroup, (int)precache);
    return check_launch();
}

}  // extern "C"
