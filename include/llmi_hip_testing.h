/*
 * llmi_hip_testing.h -- hooks of libllmi_hip.so that exist for its test suite only. They have no counterpart in
 * the reference and no use in an engine: nothing here is part of the drop-in boundary (llmi_hip.h).
 */
#ifndef LLMI_HIP_TESTING_H
#define LLMI_HIP_TESTING_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* With the workspace laid out by package side a split keeps its partial results and record in the home near its own
 * XCD, and the workgroup that merges finds them in the home near itself because both run on one XCD. `mode` 1 makes
 * every split but the merging one use the OTHER home, mode 2 every second split: what a launch would look like whose
 * workgroups were not dealt to the XCDs as expected. The merging workgroup must then find the records by its
 * fall-back (both homes, after 16 rounds of polls) and read every split's partial results from the right home: same
 * result, a few microseconds later. 0 (the default) switches it off. Applies to launches enqueued after the call;
 * returns the previous mode. */
int32_t llmi_hip_set_test_far_home(int32_t mode);

/* The decision llmi_hip_mha_workspace_side takes from one run of the ping-pong probe, as a pure function of the
 * probe's 64 result words (llmi_hip_probe_block_pingpong): 1 = XCDs 0-3 are nearer to the block with address bit 13
 * clear and XCDs 4-7 to the one with the bit set, 2 = the other way round, 0 = no statement (fewer than two usable
 * pairs on a side, or a side whose two blocks differ by less than the threshold, or both sides preferring the same
 * block). Makes no HIP call. */
int32_t llmi_hip_side_from_pingpong(const uint32_t* results64);

/* ... and how several such decisions become the measurement's answer: the side that at least two decisions name, as
 * long as no decision names the other one; else 0. *verdict (optional): 0 = agreed, 1 = abstained (fewer than two
 * statements), 2 = contradicted (both sides named). */
int32_t llmi_hip_side_agreement(const int32_t* decisions, int32_t count, int32_t* verdict);

/* What llmi_hip_mha_workspace_side has answered since the library was loaded, per 2 MiB region it measured:
 * out[0] = regions with an agreed side, out[1] = abstentions, out[2] = contradictions. */
void llmi_hip_workspace_side_stats(uint64_t out[3]);

/* The launcher's rule for the staggered walk of the split path (split s starts its walk s & mask tiles into each
 * wavefront's sequence): the mask it would use for a cache in `kv_layout` whose splits' runs are `run_bytes` long
 * (`ragged` != 0: some splits take one tile more); 0 = every split starts at its first tile. Makes no HIP call. */
int32_t llmi_hip_stagger_mask(int32_t kv_layout, int64_t run_bytes, int32_t ragged);

#ifdef __cplusplus
}
#endif
#endif /* LLMI_HIP_TESTING_H */
