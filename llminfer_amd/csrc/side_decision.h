// Which 8 KiB block of a pair lies near which side of the package: the decision taken from the ping-pong probe's
// timings, as pure host functions (no HIP call), so that they can be tested with made-up timings.
#ifndef LLMI_SIDE_DECISION_H
#define LLMI_SIDE_DECISION_H

#include <stdint.h>

namespace llmi {

// Shape of one probe run (block_pingpong_kernel): round trips per chain, chains per block.
constexpr int kPingPongs = 16, kPingPongChains = 2;
// A side of the package must find one block nearer than the other by at least this much per hand-over.
constexpr long long kSideThresholdNs = 25;

// One run of the probe: eight pairs of workgroups, pair p reporting r[8*p + 0] = the XCD of its first workgroup,
// [1] / [2] = 10 ns ticks spent on the block with address bit 13 clear / set, [3] = 1 if every number arrived,
// [5] = the XCD of its second workgroup. Returns 1 if XCDs 0-3 are nearer to the clear block and XCDs 4-7 to the set
// one, 2 for the other way round, 0 for no statement: a pair counts only if it lost nothing and shared an XCD, a side
// of the package needs two such pairs, both sides must see a difference of at least the threshold, and they must
// disagree about which block is nearer.
inline int side_from_pingpong(const uint32_t* r) {
    long long diff[2] = {0, 0};  // per side of the package: ticks through the clear block minus ticks through the set block
    int n[2] = {0, 0};
    for (int p = 0; p < 8; ++p) {
        const uint32_t* q = r + 8 * p;
        if (q[3] != 1u || q[0] != q[5] || q[0] > 7u) continue;
        const int sd = (int)(q[0] >> 2) & 1;
        diff[sd] += (long long)q[1] - (long long)q[2];
        ++n[sd];
    }
    if (n[0] < 2 || n[1] < 2) return 0;
    const long long handovers = 2ll * kPingPongs * kPingPongChains;  // two per round trip
    const long long d0 = diff[0] * 10 / (n[0] * handovers), d4 = diff[1] * 10 / (n[1] * handovers);  // ns per hand-over
    if (d0 <= -kSideThresholdNs && d4 >= kSideThresholdNs) return 1;
    if (d0 >= kSideThresholdNs && d4 <= -kSideThresholdNs) return 2;
    return 0;
}

enum SideVerdict { kSideAgreed = 0, kSideAbstained = 1, kSideContradicted = 2 };

// Several runs' decisions -> the measurement's answer: a side is reported only if at least two runs name it and no
// run names the other one.
inline int side_agreement(const int* decisions, int count, int* verdict) {
    int votes[3] = {0, 0, 0};
    for (int i = 0; i < count; ++i)
        if (decisions[i] == 1 || decisions[i] == 2) ++votes[decisions[i]];
    int v, side = 0;
    if (votes[1] && votes[2]) v = kSideContradicted;
    else if (votes[1] >= 2) v = kSideAgreed, side = 1;
    else if (votes[2] >= 2) v = kSideAgreed, side = 2;
    else v = kSideAbstained;
    if (verdict) *verdict = v;
    return side;
}

}  // namespace llmi

#endif
