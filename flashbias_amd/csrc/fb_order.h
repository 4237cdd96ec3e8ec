// Which tile of which (batch, head) unit a workgroup takes.  Plain C++ (host and device): the launch order is
// checked on the CPU by sanitize_check.cpp.
#pragma once

#if defined(__HIPCC__)
#define FB_HD __host__ __device__ __forceinline__
#else
#define FB_HD inline
#endif

namespace fb {

// Workgroup `wg` of a launch of `total` = units x ntiles workgroups takes tile `pos` of unit `unit`.  The hardware
// deals workgroup ids round-robin over the 8 XCDs and starts them in the order of their ids.  Each XCD gets one
// contiguous share of the unit-major numbering (unit * ntiles + pos), so that the workgroups of a unit meet in one
// L2.  Without a causal mask the share is walked
// in that numbering.  Under a causal mask `pos` counts a unit's tiles from the longest, a workgroup's length falls
// from ntiles to 1 key (query) tiles, and walking unit by unit ends every share with the long workgroups of its
// last unit while most of the chip has run dry (B1 H50 L=4096 in 128-row tiles: 60 tile times for a share of 200
// workgroups on 96 slots where 38 would do).  The share is therefore walked longest first: all its workgroups at
// position 0, then all at position 1, and so on; the workgroups of a unit still start within a few positions of
// each other and sweep the keys together.
FB_HD void work_order(int wg, int ntiles, int total, bool causal, int &unit, int &pos) {
    constexpr int kXcd = 8;
    // XCD x receives the ids x, x + 8, ...: total / 8 of them, one more on the first total % 8 XCDs
    const int x = wg % kXcd, j = wg / kXcd, per = total / kXcd, more = total % kXcd;
    const int w0 = x * per + (x < more ? x : more), w1 = w0 + per + (x < more ? 1 : 0);
    const int ua = w0 / ntiles, p0 = w0 % ntiles; // the share's first unit, from position p0 on
    if (!causal) {
        unit = (w0 + j) / ntiles;
        pos = (w0 + j) % ntiles;
        return;
    }
    const int ub = (w1 - 1) / ntiles, p1 = (w1 - 1) % ntiles + 1; // its last unit, positions below p1
    if (ua == ub) {
        unit = ua;
        pos = p0 + j;
        return;
    }
    const int nfull = ub - ua - 1; // units in between have every position
    // workgroups of the share at positions below p
    auto before = [&](int p) { return nfull * p + (p > p0 ? p - p0 : 0) + (p < p1 ? p : p1); };
    int lo = 0, hi = ntiles - 1; // the last position with before(position) <= j
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (before(mid) <= j)
            lo = mid;
        else
            hi = mid - 1;
    }
    pos = lo;
    const int k = j - before(lo); // among the units that have this position: [ua,] ua + 1 ... ua + nfull [, ub]
    unit = lo >= p0 ? ua + k : ua + 1 + k;
}

} // namespace fb
