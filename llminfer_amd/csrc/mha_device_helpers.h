// Device-side helpers shared by the decode-attention kernels (mha_decode_kernels.h) and the multi-layer kernel
// (mha_stack.hip): lane folds over the four DPP rows, LDS-DMA loads, the fused QK-Norm + RoPE on rows held in LDS,
// and where a query head keeps its rows of the fused combine's workspace. Everything here has internal linkage:
// every translation unit that includes it gets its own copy, including its own give-up counter.
#ifndef LLMI_MHA_DEVICE_HELPERS_H
#define LLMI_MHA_DEVICE_HELPERS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "llmi_internal.h"
#include "mha_decode_args.h"
#include "wave_ops.h"

namespace llmi {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));

namespace {


// Waits of the fused combine that ran out of polls, counted on the device (one per head and call).
__device__ unsigned int g_poll_timeouts = 0;

constexpr int kTile = 16;      // positions per MFMA tile
constexpr int kHeadDim = 128;
// Fused output projection: weight rows a wavefront holds in registers while it waits for the attention
// output, and 512-element steps per row (kOprojSteps * 512 = the widest attention output it takes).
constexpr int kOprojRows = 3;
constexpr int kOprojSteps = 8;
// Cache policy of the buffer loads and stores that hand partial results from one workgroup to
// another: the instruction's sc1 bit, device scope (served by memory, coherent across the XCDs).
constexpr int kCacheDevice = 16;
// Build-time tuning knobs.
#ifndef LLMI_NT_LOADS
#define LLMI_NT_LOADS 1  // K/V are read once: stream them past the caches
#endif
#ifndef LLMI_MIN_WAVES_PER_EU
#define LLMI_MIN_WAVES_PER_EU 2
#endif
#ifndef LLMI_OPROJ_PREFETCH_ROWS
// Weight rows (of 3 per wavefront) the fused output projection requests before it waits for the
// attention output; the others are requested after the wait.
#define LLMI_OPROJ_PREFETCH_ROWS 3
#endif
#ifndef LLMI_SPREAD_MERGE
// 1: the heads of a KV head are merged by different workgroups of the split path (see `spread` in mha_decode_body);
// 0: by the workgroup of the last split, a wavefront each. Kept for the side-by-side measurement.
#define LLMI_SPREAD_MERGE 1
#endif
#ifndef LLMI_TIMING_BARRIER_PER_TILE
// 1: a workgroup barrier in front of every tile of the decode kernel's loop (timing only: results unchanged, just slower).
#define LLMI_TIMING_BARRIER_PER_TILE 0
#endif
#ifndef LLMI_PV_VALU
// 1: the probability x value product runs on the vector ALU (fp32 multiply-adds with the
// probabilities broadcast by DPP, the structure of the reference's inner loop,
// code/source/op/kernel/cuda/mha_kernel.cu:114-155) instead of the matrix cores. Kept for the
// side-by-side measurement that decides between the two; the library is built with 0.
#define LLMI_PV_VALU 0
#endif


template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// Value of lane SRC of the caller's 16-lane DPP row.
template <int SRC>
__device__ __forceinline__ float row_bcast(float x) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x150 + SRC, 0xf, 0xf, false));
}

// Value of lane 4*k + R of the caller's own 16-lane DPP row, k = the row's number: four row broadcasts, each
// enabled for one row only (the DPP row mask), so the source lane differs from row to row without a trip through
// the LDS crossbar.
template <int R>
__device__ __forceinline__ float row_bcast_per_row(float x) {
    const int xi = __builtin_bit_cast(int, x);
    int y = __builtin_amdgcn_update_dpp(0, xi, 0x150 + R, 0x1, 0xf, false);
    y = __builtin_amdgcn_update_dpp(y, xi, 0x150 + 4 + R, 0x2, 0xf, false);
    y = __builtin_amdgcn_update_dpp(y, xi, 0x150 + 8 + R, 0x4, 0xf, false);
    y = __builtin_amdgcn_update_dpp(y, xi, 0x150 + 12 + R, 0x8, 0xf, false);
    return __builtin_bit_cast(float, y);
}

// Folds over lanes l, l^16, l^32, l^48 (the four DPP rows), the result in all of them, with the
// gfx950 lane swaps: v_permlane32_swap / v_permlane16_swap of a register with itself leave the
// lower-half (even-row) values in one result and the upper-half (odd-row) values in the other,
// each in both places. Plain VALU instructions: no trip through the LDS crossbar like a shuffle.
__device__ __forceinline__ float rows_max(float x) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    const auto h = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned h0 = h[0], h1 = h[1];
    const float y = fmaxf(__builtin_bit_cast(float, h0), __builtin_bit_cast(float, h1));
    const unsigned v = __builtin_bit_cast(unsigned, y);
    const auto q = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    const unsigned q0 = q[0], q1 = q[1];
    return fmaxf(__builtin_bit_cast(float, q0), __builtin_bit_cast(float, q1));
}
// x[l] + x[l ^ 32] in both lanes.
__device__ __forceinline__ float halves_sum(float x) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    const auto h = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned h0 = h[0], h1 = h[1];
    return __builtin_bit_cast(float, h0) + __builtin_bit_cast(float, h1);
}
__device__ __forceinline__ float rows_sum(float x) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    const auto h = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned h0 = h[0], h1 = h[1];
    const float y = __builtin_bit_cast(float, h0) + __builtin_bit_cast(float, h1);
    const unsigned v = __builtin_bit_cast(unsigned, y);
    const auto q = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    const unsigned q0 = q[0], q1 = q[1];
    return __builtin_bit_cast(float, q0) + __builtin_bit_cast(float, q1);
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }

// Round to nearest even, NaN kept quiet.
__device__ __forceinline__ uint16_t f32_to_bf16(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    if (x != x) return 0x7fc0;
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Two floats rounded to nearest even into one dword of bf16 (lo = a, hi = b).
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
}

// 16 bytes per lane from global memory straight into LDS, no VGPR round trip:
// lane L's bytes land at lds_off + 16*L. `base` and `lds_off` are wave-uniform,
// `voff` is the lane's byte offset from base. Counted by vmcnt like any load.
__device__ __forceinline__ void dma16(const char* base, uint32_t voff, uint32_t lds_off) {
    // The instruction takes its base and the LDS offset (through M0) from scalar
    // registers; readfirstlane guarantees that whatever the surrounding code
    // made of these wave-uniform values (it is free when they already are scalar).
    // M0 is an operand of the asm statement (constraint {m0}): the compiler writes it and
    // knows that it is live; the s_nop covers the wait state between that write and the load.
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    // (the builtin returns a signed int: go through uint32_t so that the low half is not sign-extended)
    const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b);
    const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
    const uint64_t sbase = ((uint64_t)b_hi << 32) | (uint64_t)b_lo;
    const uint32_t slds = (uint32_t)__builtin_amdgcn_readfirstlane(lds_off);
#if LLMI_NT_LOADS
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt" :: "v"(voff), "s"(sbase), "{m0}"(slds) : "memory");
#else
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" :: "v"(voff), "s"(sbase), "{m0}"(slds) : "memory");
#endif
}

// Same, with a full 64-bit address per lane and without the streaming hint: for small
// operands that many workgroups share (they stay in L2).
__device__ __forceinline__ void dma16_gather(const void* ptr, uint32_t lds_off) {
    const uint32_t slds = (uint32_t)__builtin_amdgcn_readfirstlane(lds_off);
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(ptr), "{m0}"(slds) : "memory");
}

// Same, device scope (sc1: served by memory, past the L2 of the XCD the wavefront runs on): for data another
// workgroup of the same launch has written.
__device__ __forceinline__ void dma16_gather_coherent(const void* ptr, uint32_t lds_off) {
    const uint32_t slds = (uint32_t)__builtin_amdgcn_readfirstlane(lds_off);
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off sc1" :: "v"(ptr), "{m0}"(slds) : "memory");
}

// Waits until at most `newer_tiles` whole tiles (8 loads each) are still in flight.
__device__ __forceinline__ void wait_tiles_in_flight(int newer_tiles) {
    if (newer_tiles <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (newer_tiles == 1) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else if (newer_tiles == 2) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
}

struct TileRegs {
    u32x4 k[4];
    u32x4 v[4];
};

// What the attention part of an OPROJ kernel hands to the projection part.
struct OprojState {
    uint32_t gen_base = 0u;  // the generation word as read before this workgroup published anything
    bool worker = false;     // this workgroup takes rows of the projection (it is not a combiner)
};

// Where a query head keeps its rows of the fused combine's partial and record arrays.
// The eight XCDs sit on two sides of the package, and so does memory: which side an address belongs to
// changes every 8 KiB (address bit 13, hashed with higher bits: the same within a 2 MiB-aligned region, different
// between regions), and a store -> poll -> load hand-over between workgroups of one XCD takes 0.1-0.2 us longer
// through the far side than through the near one (the ping-pong probe shows it per XCD and block). With a.by_side
// every row therefore has two homes, one in each 8 KiB block of a 16 KiB-aligned pair, and a workgroup uses the home
// near the XCD it finds itself on (hardware id register): a split stores its partial outputs and its record there,
// the combiner polls the records' home near itself and reads a split's partial outputs from the home that goes with
// the one it found the record in. With the KV head in blockIdx.x and a KV head count that is a multiple of eight, all
// workgroups of a KV head run on one XCD (they are dealt to the XCDs in turn), so they agree on the home and
// everything they hand over travels through near memory. Nothing relies on that placement for its result: after 16
// rounds of polls the combiner also looks into the other home for the records it is still missing, so a split that
// ran on the other side is found later, not never. Which block of a pair is near which side is what
// llmi_hip_mha_workspace_side measures, per 2 MiB region; the launcher turns it into one bit per head and array.
struct WsHead {
    int rbase;     // the head's first row: head * num_splits
    bool by_side;
    int ppar, rpar;  // partials / records: which block of a pair (address bit 13) side 0 of the package uses for this head
};
// BYSIDE is a kernel's compile-time choice: the plain layout's instantiations carry none of the other's code.
template <bool BYSIDE>
__device__ __forceinline__ WsHead ws_head(const KernelArgs& a, int hq) {
    WsHead w{hq * a.num_splits, BYSIDE, 0, 0};
    if constexpr (BYSIDE) {
        w.ppar = (int)(((hq < 64 ? a.ppar[0] : a.ppar[1]) >> (hq & 63)) & 1ull);
        w.rpar = (int)(((hq < 64 ? a.rpar[0] : a.rpar[1]) >> (hq & 63)) & 1ull);
    }
    return w;
}
// Row of split sp in the home that a workgroup on side xs of the package (0: XCDs 0-3, 1: XCDs 4-7) uses:
// SH = 4 for the partials (16 rows of 512 bytes per 8 KiB block), 9 for the records (512 of 16 bytes).
template <int SH>
__device__ __forceinline__ int ws_row(const WsHead& w, int sp, int xs) {
    const int r = w.rbase + sp;
    if (!w.by_side) return r;
    const int parity = (SH == 4 ? w.ppar : w.rpar) ^ xs;  // bit 13 of the home's address (a pair starts on a 16 KiB boundary)
    return ((((r >> SH) << 1) + parity) << SH) + (r & ((1 << SH) - 1));
}
constexpr uint32_t kSideBlockBytes = 8192u;
// Side of the package this workgroup's XCD is on (0 in the plain layout).
template <bool BYSIDE>
__device__ __forceinline__ int package_side() {
    if constexpr (!BYSIDE) return 0;
    uint32_t xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    return (int)((xcc >> 2) & 1u);
}

// RMSNorm * weight + half-rotation RoPE of 128-wide bf16 rows held in LDS, in place, by one
// wavefront: the 16 lanes of DPP row r take row `row` of `rows` (256 bytes each); lane p of them
// takes elements 4*(p&1) .. +3 of 16-byte chunk p>>1 and of its rotary partner, chunk (p>>1) + 8,
// so a lane touches 8 elements, reads only what it overwrites, and the sum of squares is one
// DPP row fold. `w`: the 256-byte norm weights; `sin16` / `cos16`: the 64 sines / cosines of the
// position (lane p needs exactly 16-byte chunk p of each). Same chain as the stand-alone kernel
// (x*w*r, then a*cos - b*sin / a*sin + b*cos on the pairs (i, i+64)), rounded to bf16 once.
__device__ __forceinline__ void norm_rope_rows_lds(char* rows, const char* w, const char* sin16, const char* cos16,
                                                   int row, int p, float eps) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const int c = p >> 1, hf = p & 1;
    u32x2* lo_p = reinterpret_cast<u32x2*>(rows + (row * 16 + c) * 16 + hf * 8);
    u32x2* hi_p = reinterpret_cast<u32x2*>(rows + (row * 16 + c + 8) * 16 + hf * 8);
    const u32x2 xl = *lo_p, xh = *hi_p;
    const u32x2 wl = *reinterpret_cast<const u32x2*>(w + c * 16 + hf * 8);
    const u32x2 wh = *reinterpret_cast<const u32x2*>(w + (c + 8) * 16 + hf * 8);
    const f32x4 sn = *reinterpret_cast<const f32x4*>(sin16 + p * 16);
    const f32x4 cs = *reinterpret_cast<const f32x4*>(cos16 + p * 16);
    const uint32_t xl0 = xl[0], xl1 = xl[1], xh0 = xh[0], xh1 = xh[1];
    const uint32_t wl0 = wl[0], wl1 = wl[1], wh0 = wh[0], wh1 = wh[1];
    const float a[4] = {bf16_lo(xl0), bf16_hi(xl0), bf16_lo(xl1), bf16_hi(xl1)};
    const float b[4] = {bf16_lo(xh0), bf16_hi(xh0), bf16_lo(xh1), bf16_hi(xh1)};
    const float wa[4] = {bf16_lo(wl0), bf16_hi(wl0), bf16_lo(wl1), bf16_hi(wl1)};
    const float wb[4] = {bf16_lo(wh0), bf16_hi(wh0), bf16_lo(wh1), bf16_hi(wh1)};
    float ss = 0.0f;
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += a[e] * a[e];
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += b[e] * b[e];
    ss += dpp_partner<0xB1>(ss);
    ss += dpp_partner<0x4E>(ss);
    ss += dpp_partner<0x141>(ss);
    ss += dpp_partner<0x140>(ss);
    const float r = 1.0f / sqrtf(ss / (float)kHeadDim + eps);
    float ol[4], oh[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float av = a[e] * wa[e] * r;
        const float bv = b[e] * wb[e] * r;
        ol[e] = av * cs[e] - bv * sn[e];
        oh[e] = av * sn[e] + bv * cs[e];
    }
    *lo_p = u32x2{pack_bf16(ol[0], ol[1]), pack_bf16(ol[2], ol[3])};
    *hi_p = u32x2{pack_bf16(oh[0], oh[1]), pack_bf16(oh[2], oh[3])};
}

}  // namespace
}  // namespace llmi

#endif
