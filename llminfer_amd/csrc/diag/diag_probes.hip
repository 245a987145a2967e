// Diagnostic kernels of libllmi_diag.so (declared in llmi_hip_diag.h): how a value stored by one workgroup becomes
// visible to a polling workgroup under every pair of store / load cache policies, and where the workgroups of a
// launch with a decode workgroup's footprint land. They answered design questions of the decode kernel's hand-over;
// nothing in libllmi_hip.so or the host layer uses them, only bench.py's two diagnostic modes and their tests.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "llmi_hip.h"
#include "llmi_hip_diag.h"

namespace {

__device__ __forceinline__ uint32_t xcc_id() {
    uint32_t x;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
    return x & 15u;
}

template <int M>
__device__ __forceinline__ uint32_t load_policy(const uint32_t* p) {
    uint32_t v;
    if constexpr (M == LLMI_DIAG_PLAIN) asm volatile("global_load_dword %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    if constexpr (M == LLMI_DIAG_SC0) asm volatile("global_load_dword %0, %1, off sc0\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    if constexpr (M == LLMI_DIAG_SC1) asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    if constexpr (M == LLMI_DIAG_SC0_SC1) asm volatile("global_load_dword %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    if constexpr (M == LLMI_DIAG_NT) asm volatile("global_load_dword %0, %1, off nt\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    return v;
}
template <int M>
__device__ __forceinline__ void store_policy(uint32_t* p, uint32_t v) {
    if constexpr (M == LLMI_DIAG_PLAIN) asm volatile("global_store_dword %0, %1, off\n\ts_waitcnt vmcnt(0)" ::"v"(p), "v"(v) : "memory");
    if constexpr (M == LLMI_DIAG_SC0) asm volatile("global_store_dword %0, %1, off sc0\n\ts_waitcnt vmcnt(0)" ::"v"(p), "v"(v) : "memory");
    if constexpr (M == LLMI_DIAG_SC1) asm volatile("global_store_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" ::"v"(p), "v"(v) : "memory");
    if constexpr (M == LLMI_DIAG_SC0_SC1) asm volatile("global_store_dword %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" ::"v"(p), "v"(v) : "memory");
    if constexpr (M == LLMI_DIAG_NT) asm volatile("global_store_dword %0, %1, off nt\n\ts_waitcnt vmcnt(0)" ::"v"(p), "v"(v) : "memory");
}

constexpr uint32_t kProbeValue = 42u;
constexpr uint32_t kProbePolls = 4000u;

// line[0]: the data word; line[64] (another 256-byte line): reader -> writer "I am polling".
template <int WM, int RM>
__global__ __launch_bounds__(64) void handover_kernel(uint32_t* line, llmi_diag_handover_result* res, int writer_wg, int reader_wg, int precache) {
    if (threadIdx.x != 0) return;
    uint32_t* data = line;
    uint32_t* flag = line + 64;
    if ((int)blockIdx.x == reader_wg) {
        if (precache) (void)(load_policy<LLMI_DIAG_PLAIN>(data) + load_policy<RM>(data));
        store_policy<LLMI_DIAG_SC1>(flag, 1u);
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
            if (load_policy<LLMI_DIAG_SC1>(flag) == 1u) break;
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

typedef void (*HandoverKernel)(uint32_t*, llmi_diag_handover_result*, int, int, int);
template <int WM>
HandoverKernel pick_reader(int rm) {
    switch (rm) {
        case LLMI_DIAG_PLAIN: return handover_kernel<WM, LLMI_DIAG_PLAIN>;
        case LLMI_DIAG_SC0: return handover_kernel<WM, LLMI_DIAG_SC0>;
        case LLMI_DIAG_SC1: return handover_kernel<WM, LLMI_DIAG_SC1>;
        case LLMI_DIAG_SC0_SC1: return handover_kernel<WM, LLMI_DIAG_SC0_SC1>;
        default: return handover_kernel<WM, LLMI_DIAG_NT>;
    }
}

int check(hipError_t e) { return e == hipSuccess ? LLMI_OK : LLMI_ERR_LAUNCH; }

}  // namespace

extern "C" {

int llmi_diag_placement(int32_t workgroups, int32_t exclusive, uint32_t* ids, void* stream) {
    if (!ids) return LLMI_ERR_NULL_POINTER;
    if (workgroups < 1 || workgroups > 4096) return LLMI_ERR_INVALID_ARG;
    if ((uintptr_t)ids & 3u) return LLMI_ERR_ALIGNMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint32_t hold = 500;  // 5 us
    if (exclusive) hipLaunchKernelGGL((placement_kernel<84 * 1024>), dim3(workgroups), dim3(256), 0, s, ids, hold);
    else hipLaunchKernelGGL((placement_kernel<66 * 1024>), dim3(workgroups), dim3(256), 0, s, ids, hold);
    return check(hipGetLastError());
}

int llmi_diag_handover(int32_t store_pol, int32_t load_pol, int32_t writer_workgroup, int32_t reader_workgroup, int32_t precache, void* line,
                            llmi_diag_handover_result* result, void* stream) {
    if (!line || !result) return LLMI_ERR_NULL_POINTER;
    if (store_pol < 0 || store_pol > LLMI_DIAG_NT || load_pol < 0 || load_pol > LLMI_DIAG_NT) return LLMI_ERR_INVALID_ARG;
    if (writer_workgroup < 0 || writer_workgroup > 15 || reader_workgroup < 0 || reader_workgroup > 15 || writer_workgroup == reader_workgroup)
        return LLMI_ERR_INVALID_ARG;
    if ((uintptr_t)line & 255u) return LLMI_ERR_ALIGNMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (int rc = check(hipMemsetAsync(line, 0, 4096, s))) return rc;
    if (int rc = check(hipMemsetAsync(result, 0, sizeof(*result), s))) return rc;
    HandoverKernel k;
    switch (store_pol) {
        case LLMI_DIAG_PLAIN: k = pick_reader<LLMI_DIAG_PLAIN>(load_pol); break;
        case LLMI_DIAG_SC0: k = pick_reader<LLMI_DIAG_SC0>(load_pol); break;
        case LLMI_DIAG_SC1: k = pick_reader<LLMI_DIAG_SC1>(load_pol); break;
        case LLMI_DIAG_SC0_SC1: k = pick_reader<LLMI_DIAG_SC0_SC1>(load_pol); break;
        default: k = pick_reader<LLMI_DIAG_NT>(load_pol); break;
    }
    hipLaunchKernelGGL(k, dim3(16), dim3(64), 0, s, static_cast<uint32_t*>(line), result, (int)writer_workgroup, (int)reader_workgroup, (int)precache);
    return check(hipGetLastError());
}

}  // extern "C"
