// Which claim counter a workgroup serves and which tiles that counter owns, shared by the device
// dispatcher (csrc/tile_loop.hpp) and the host-side accounting (BLPExecutor::read_counters).
//
// MI355X has 8 XCDs, each with its own L2; the hardware hands consecutive workgroups of a launch
// to consecutive XCDs (workgroup b runs on XCD b % 8).  Tiles that sit next to each other in the
// tile order share operand rows, so a counter's slice should be worked on by one XCD, and the
// slices of one XCD should be adjacent: then an operand block is fetched into few L2s instead of
// all eight.  With `groups` a multiple of 8, group g is therefore served by the workgroups
//     b % 8 == g / (groups/8)   and   (b / 8) % (groups/8) == g % (groups/8),
// so groups [k*groups/8, (k+1)*groups/8) belong to XCD k.  Fewer than 8 groups fall back to
// b % groups.  Slice sizes are proportional to the number of workgroups serving the group, so a
// launch with one workgroup per tile gives every workgroup exactly one tile.
#pragma once

#if defined(__HIPCC__)
#define GP_HD __host__ __device__ inline
#else
#define GP_HD inline
#endif

namespace gp {

constexpr int kXcds = 8;

// `groups` is a power of two (the launchers refuse anything else).  Everything below is evaluated
// by every wavefront at the start of a kernel, in front of its first memory access, so it avoids
// divisions by run-time values: shifts and masks for the group arithmetic, and one 32-bit division
// for the slice boundary whenever the product fits (a 64-bit division is about 200 instructions
// on this hardware, and two of them plus the divisions of the loop below used to add almost 2 us
// to every preemptible launch).
GP_HD int log2_pow2(int v) { return __builtin_ctz((unsigned)v); }

GP_HD int wg_group(int b, int groups) {
    if (groups <= 1) return 0;
    if (groups < kXcds) return b & (groups - 1);
    const int per = groups / kXcds;  // a constant shift: kXcds is a compile-time power of two
    return (b % kXcds) * per + ((b / kXcds) & (per - 1));
}

// number of workgroups (of a grid of `grid`) that serve groups [0, g)
GP_HD long group_wgs_before(int g, int groups, int grid) {
    if (groups <= 1) return g > 0 ? grid : 0;
    const int lg = log2_pow2(groups);
    const int q = grid >> lg, r = grid & (groups - 1);
    if (groups < kXcds) return (long)g * q + (g < r ? g : r);
    // group g' = k*per + a is first served by workgroup w0 = 8*a + k and has one workgroup more
    // than q when w0 < r.  Count those among g' < g, residue a at a time.
    const int per = groups / kXcds, lper = lg - 3;
    long extra = 0;
    for (int a = 0; a < per; ++a) {
        int by_r = r - kXcds * a;                  // k < r - 8a
        int by_g = (g - a + per - 1) >> lper;      // k*per + a < g   (g - a + per - 1 >= 0)
        int c = by_r < by_g ? by_r : by_g;
        if (c > kXcds) c = kXcds;
        if (c > 0) extra += c;
    }
    return (long)g * q + extra;
}

// first tile (in tile order) of group g's slice: floor(total * workgroups before g / grid)
GP_HD int group_slice_begin(int total, int g, int groups, int grid) {
    const unsigned long long prod = (unsigned long long)total * (unsigned long long)group_wgs_before(g, groups, grid);
    if (prod <= 0xFFFFFFFFull) return (int)((unsigned)prod / (unsigned)grid);
    return (int)(prod / (unsigned long long)grid);
}

// A launch with several counters and at least as many workgroups as claims does not hand claims
// out through the counters: workgroup b takes claim xcd_contiguous(b, total) and records it as bit
// b / groups in ints 1..15 of the 16-int line of counter wg_group(b, groups); int 0 of each line
// counts the claims made (see csrc/tile_loop.hpp).  The slices above play no part then.
constexpr int kFixedClaimBits = 15 * 32;
GP_HD bool fixed_claims(bool counters, int groups, int grid, int total) {
    return counters && groups > 1 && grid >= total && grid <= groups * kFixedClaimBits;
}

// Launches without claim counters (one workgroup per tile): workgroup b takes tile order index
// xcd_contiguous(b, total), which gives XCD k the contiguous range of the tile order that its
// workgroups b = k, k+8, ... cover.
GP_HD int xcd_contiguous(int b, int total) {
    const int k = b % kXcds, i = b / kXcds;
    const int q = total / kXcds, r = total % kXcds;
    return k * q + (k < r ? k : r) + i;
}

}  // namespace gp
