// CPU check of include/util/slice_map.h: the slices partition the tile order, their sizes follow
// the number of workgroups that serve them, and the static mapping is a bijection.
#include <cstdio>
#include <vector>
#include "util/slice_map.h"

int main() {
    long cases = 0;
    const int group_counts[] = {1, 2, 4, 8, 16, 32, 64};
    for (int groups : group_counts)
        for (int grid = groups; grid <= 600; grid += (grid < 80 ? 1 : 37))
            for (int total : {grid, grid + 1, 3 * grid + 5, 1, 7, 392, 1024, 4096, 100000}) {
                // workgroups per group, by enumeration
                std::vector<long> cnt(groups, 0);
                for (int b = 0; b < grid; ++b) {
                    int g = gp::wg_group(b, groups);
                    if (g < 0 || g >= groups) { printf("wg_group out of range: b=%d groups=%d -> %d\n", b, groups, g); return 1; }
                    cnt[g]++;
                }
                long before = 0;
                int prev_begin = 0;
                for (int g = 0; g <= groups; ++g) {
                    if (gp::group_wgs_before(g, groups, grid) != before) {
                        printf("wgs_before mismatch groups=%d grid=%d g=%d: %ld vs %ld\n", groups, grid, g, gp::group_wgs_before(g, groups, grid), before);
                        return 1;
                    }
                    int begin = gp::group_slice_begin(total, g, groups, grid);
                    if (begin < prev_begin) { printf("slices not monotone\n"); return 1; }
                    if (g == 0 && begin != 0) { printf("first slice does not start at 0\n"); return 1; }
                    if (g == groups && begin != total) { printf("last slice does not end at total\n"); return 1; }
                    prev_begin = begin;
                    if (g < groups) before += cnt[g];
                }
                if (total == grid)  // one workgroup per tile: every group's slice equals its workgroup count
                    for (int g = 0; g < groups; ++g)
                        if (gp::group_slice_begin(total, g + 1, groups, grid) - gp::group_slice_begin(total, g, groups, grid) != cnt[g]) {
                            printf("slice size != workgroups: groups=%d grid=%d g=%d\n", groups, grid, g);
                            return 1;
                        }
                ++cases;
            }
    // groups of one XCD are adjacent and served by that XCD only
    for (int b = 0; b < 4096; ++b)
        if (gp::wg_group(b, 32) / 4 != b % 8) { printf("group %d of workgroup %d is not on XCD %d\n", gp::wg_group(b, 32), b, b % 8); return 1; }
    for (int total = 1; total <= 3000; ++total) {
        std::vector<char> seen(total, 0);
        int last[8] = {-1, -1, -1, -1, -1, -1, -1, -1};
        for (int b = 0; b < total; ++b) {
            int u = gp::xcd_contiguous(b, total);
            if (u < 0 || u >= total || seen[u]) { printf("xcd_contiguous not a bijection: total=%d b=%d u=%d\n", total, b, u); return 1; }
            seen[u] = 1;
            if (last[b % 8] >= 0 && u != last[b % 8] + 1) { printf("XCD range not contiguous: total=%d b=%d\n", total, b); return 1; }
            last[b % 8] = u;
        }
    }
    // fixed claims: workgroup b records its claim as bit (b / groups) of counter wg_group(b); the
    // pairs must be distinct over a grid and the bit must fit the 15 spare ints of a counter's line
    for (int groups : {8, 16, 32, 64})
        for (int grid : {groups, 100, 392, 396, 1572, 2048, groups * gp::kFixedClaimBits}) {
            if (grid < groups) continue;
            if (!gp::fixed_claims(true, groups, grid, grid) || gp::fixed_claims(true, groups, grid, grid + 1) ||
                gp::fixed_claims(false, groups, grid, grid) || gp::fixed_claims(true, 1, grid, grid) ||
                gp::fixed_claims(true, groups, groups * gp::kFixedClaimBits + 1, grid)) {
                printf("fixed_claims predicate wrong: groups=%d grid=%d\n", groups, grid);
                return 1;
            }
            std::vector<char> seen((size_t)groups * gp::kFixedClaimBits, 0);
            for (int b = 0; b < grid; ++b) {
                int g = gp::wg_group(b, groups), j = b >> gp::log2_pow2(groups);
                if (j >= gp::kFixedClaimBits || seen[(size_t)g * gp::kFixedClaimBits + j]) {
                    printf("claim bit reused or out of range: groups=%d grid=%d b=%d\n", groups, grid, b);
                    return 1;
                }
                seen[(size_t)g * gp::kFixedClaimBits + j] = 1;
            }
            ++cases;
        }
    printf("ok %ld cases\n", cases);
    return 0;
}
