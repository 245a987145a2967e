/*
 * llmi_hip_probes.h -- measurement kernels of libllmi_hip.so. They have no counterpart in the reference
 * and compute nothing a model needs: bench.py uses them to put a floor under the decode-attention
 * figures (what the machine does with the same bytes when nothing is computed) and to calibrate HBM byte
 * counters; llmi_hip_mha_workspace_side decides on the ping-pong probe.
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

/* The decode kernel's K/V stream without its arithmetic, one feature at a time, on the decode kernel's own grid
 * (kv_heads x splits workgroups, the KV head fastest; a head's 16-position tiles dealt to splits and wavefronts as the
 * decode kernel deals them). `k`, `v`: caches of `positions` positions (a multiple of 16) of `kv_heads` heads x 256
 * bytes in `kv_layout` (LLMI_KV_LAYOUT_*). (waves, tiles_in_flight) one of (4,2), (8,1), (8,2), (4,4). `mode`:
 * 0 = ordinary non-temporal loads to registers; 1 = LDS-DMA loads into per-wavefront rings, whole rows per
 * instruction; 2 = 1 with the K chunks swizzled by row & 7, exactly the decode kernel's requests; 3 = 2 with a pause
 * of `pause` x 64 clocks (0..1024) after every tile has landed, standing for the arithmetic. `stagger` (0..255):
 * split s starts its walk s & mask tiles into each wavefront's sequence, mask = 3 if bit 0 is set, else stagger >> 2
 * (the decode kernel's choice for some lengths: 3 position-major, 31 head-major); bit 1: the grid is splits x kv_heads
 * with the split fastest (consecutive workgroups read consecutive runs of a head), not the decode kernel's order.
 * Everything read is thrown away; `sink` (>= 4 bytes, device) is never written in practice. */
int llmi_hip_probe_stream_tiles(const void* k, const void* v, int32_t positions, int32_t kv_heads, int32_t kv_layout, int32_t splits,
                                int32_t waves, int32_t tiles_in_flight, int32_t mode, int32_t pause, int32_t stagger, void* sink,
                                void* stream);

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

#ifdef __cplusplus
}
#endif
#endif /* LLMI_HIP_PROBES_H */
