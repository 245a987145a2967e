/*
 * llmi_hip_diag.h -- diagnostic kernels, in a library of their own (libllmi_diag.so): they answered two design
 * questions of the decode kernel's hand-over between workgroups (which cache policies make a store visible to a
 * polling workgroup, and where the workgroups of a launch land) and are kept so that the measurements can be
 * repeated (bench.py --handover-probe, --placement). No counterpart in the reference; libllmi_hip.so and the host
 * layer do not use them. Same conventions as llmi_hip.h: plain pointers and sizes, LLMI_OK or a negative
 * llmi_status, nothing allocated, everything enqueued on the caller's stream.
 */
#ifndef LLMI_HIP_DIAG_H
#define LLMI_HIP_DIAG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Where the workgroups of a launch land. `workgroups` (1..4096) workgroups of 256 threads with the LDS footprint of a
 * decode workgroup (66 KiB; `exclusive` != 0: 84 KiB, more than half a CU's LDS, so that no two share a CU) each write
 * ids[2*i] = the XCD and ids[2*i+1] = the hardware id register (HW_REG_HW_ID: CU, shader array and shader engine in
 * bits 8..15) of the CU they run on, and keep that CU for 5 us. `ids`: 2 * workgroups uint32 of device memory. */
int llmi_diag_placement(int32_t workgroups, int32_t exclusive, uint32_t* ids, void* stream);

/* Cache policy of one 4-byte load or store of the hand-over probe: the instruction's sc0 / sc1 / nt bits. */
enum { LLMI_DIAG_PLAIN = 0, LLMI_DIAG_SC0 = 1, LLMI_DIAG_SC1 = 2, LLMI_DIAG_SC0_SC1 = 3, LLMI_DIAG_NT = 4 };

typedef struct llmi_diag_handover_result {
    uint32_t seen;      /* 1: the reader saw the writer's value within its poll budget                      */
    uint32_t polls;     /* polls the reader made before it saw the value (or its budget, 4000)              */
    uint32_t ns;        /* reader's time from "I am polling" to "seen", 10 ns resolution; includes the
                           2 us the writer waits on purpose before it stores                                */
    uint32_t xcc_reader, xcc_writer; /* XCD each side ran on (hardware id register)                        */
} llmi_diag_handover_result;

/* One writer workgroup (`writer_workgroup`, 0..15, of a grid of 16) stores a value with `store_policy`, one reader
 * workgroup (`reader_workgroup`, 0..15, another one) polls for it with `load_policy`, a bounded number of times. When
 * workgroups are dealt to the XCDs in turn, workgroups w and w + 8 share an XCD and w + 1 is on the next one. With
 * `precache` the reader has read the line before the writer writes, so stale copies exist in its L1 and L2. `line` is
 * 4 KiB of device scratch, `result` device memory; both are overwritten. Every loop in the kernel is bounded. */
int llmi_diag_handover(int32_t store_policy, int32_t load_policy, int32_t writer_workgroup, int32_t reader_workgroup,
                            int32_t precache, void* line, llmi_diag_handover_result* result, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LLMI_HIP_DIAG_H */
