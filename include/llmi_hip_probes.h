/*
 * llmi_hip_probes.h -- measurement kernels of libllmi_hip.so. They have no counterpart in the reference
 * and compute nothing a model needs: bench.py uses them to put a floor under the decode-attention
 * figures (what the machine does with the same bytes when nothing is computed), to calibrate HBM byte
 * counters, and to show how a value written by one workgroup becomes visible to another.
 * Same conventions as llmi_hip.h: plain pointers and sizes, LLMI_OK or a negative llmi_status, nothing
 * allocated, everything enqueued on the caller's stream.
 */
#ifndef LLMI_HIP_PROBES_H
#define LLMI_HIP_PROBES_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Reads `bytes_each` bytes of `a` and of `b` exactly once (the K and V rows of a decode-attention call) with
 * the access pattern of the decode kernel's stream -- non-temporal 16-byte loads, 1 KiB per wavefront
 * instruction, 4 KiB tiles dealt to the wavefronts of a workgroup in turn, every workgroup a contiguous
 * share -- and throws them away. workgroups >= 1; waves 1, 2, 4 or 8 per workgroup; tiles_in_flight 1, 2 or 4
 * per wavefront; bytes_each a multiple of 4096. `sink` (>= 4 bytes, device) is never written in practice. */
int llmi_hip_probe_stream_read(const void* a, const void* b, size_t bytes_each, int32_t workgroups, int32_t waves,
                               int32_t tiles_in_flight, void* sink, void* stream);

/* The same stream in the position-major cache layout: `a` and `b` hold `rows` rows of `heads` x 256 bytes (a KV head's
 * part of a row is 256 bytes at offset 256 * head); the grid is (heads, workgroups_per_head), workgroup (h, g) reads head
 * h's pieces of a contiguous run of 16-row tiles, four rows per load instruction. rows a multiple of 16,
 * workgroups_per_head <= rows / 16; waves and tiles_in_flight as above. */
int llmi_hip_probe_stream_read_rows(const void* a, const void* b, int32_t rows, int32_t heads, int32_t workgroups_per_head,
                                    int32_t waves, int32_t tiles_in_flight, void* sink, void* stream);

/* dst[i] = src[i] for `bytes` bytes (a multiple of 16) with one plain kernel: reads `bytes`, writes `bytes`.
 * The known traffic the FETCH_SIZE / WRITE_SIZE counters are scaled by. */
int llmi_hip_probe_copy(const void* src, void* dst, size_t bytes, void* stream);

/* Hand-over latency from every XCD through two blocks of memory. Workgroups i and i + 8 of a grid of 16 (one XCD when
 * workgroups are dealt to the XCDs in turn) play ping-pong through their own 256-byte line of `a` (2 KiB, 256-byte
 * aligned, device), then of `b`, twice 16 round trips each, with device-scope stores and polls; every poll loop is
 * bounded. out[8*i + 0] = the XCD pair i's first workgroup ran on, [1] / [2] = 10 ns ticks spent on a / on b, [3] = 1 if
 * every number arrived, [5] = the XCD of the pair's second workgroup. `out`: 64 uint32 of device memory. Both blocks and
 * `out` are overwritten. What llmi_hip_mha_workspace_side decides on. */
int llmi_hip_probe_block_pingpong(void* a, void* b, uint32_t* out, void* stream);

/* Where the workgroups of a launch land. `workgroups` (1..4096) workgroups of 256 threads with the LDS footprint of a
 * decode workgroup (66 KiB; `exclusive` != 0: 84 KiB, more than half a CU's LDS, so that no two share a CU) each write
 * ids[2*i] = the XCD and ids[2*i+1] = the hardware id register (HW_REG_HW_ID: CU, shader array and shader engine in
 * bits 8..15) of the CU they run on, and keep that CU for 5 us. `ids`: 2 * workgroups uint32 of device memory. */
int llmi_hip_probe_placement(int32_t workgroups, int32_t exclusive, uint32_t* ids, void* stream);

/* Cache policy of one 4-byte load or store of the hand-over probe: the instruction's sc0 / sc1 / nt bits. */
enum { LLMI_PROBE_PLAIN = 0, LLMI_PROBE_SC0 = 1, LLMI_PROBE_SC1 = 2, LLMI_PROBE_SC0_SC1 = 3, LLMI_PROBE_NT = 4 };

typedef struct llmi_probe_handover_result {
    uint32_t seen;      /* 1: the reader saw the writer's value within its poll budget                      */
    uint32_t polls;     /* polls the reader made before it saw the value (or its budget, 4000)              */
    uint32_t ns;        /* reader's time from "I am polling" to "seen", 10 ns resolution; includes the
                           2 us the writer waits on purpose before it stores                                */
    uint32_t xcc_reader, xcc_writer; /* XCD each side ran on (hardware id register)                        */
} llmi_probe_handover_result;

/* One writer workgroup (`writer_workgroup`, 0..15, of a grid of 16) stores a value with `store_policy`, one reader
 * workgroup (`reader_workgroup`, 0..15, another one) polls for it with `load_policy`, a bounded number of times. When
 * workgroups are dealt to the XCDs in turn, workgroups w and w + 8 share an XCD and w + 1 is on the next one. With
 * `precache` the reader has read the line before the writer writes, so stale copies exist in its L1 and L2. `line` is
 * 4 KiB of device scratch, `result` device memory; both are overwritten. Every loop in the kernel is bounded. */
int llmi_hip_probe_handover(int32_t store_policy, int32_t load_policy, int32_t writer_workgroup, int32_t reader_workgroup,
                            int32_t precache, void* line, llmi_probe_handover_result* result, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LLMI_HIP_PROBES_H */
