// Workgroup -> tile mapping shared by the dhconv kernels.
#pragma once
#include "sfno_internal.h"

namespace sfno {

// Workgroup -> (degree, column block, row group).  Workgroups go to the 8 XCDs round-robin by linear id.  All column
// blocks and row groups of a degree share its activation panel, and the row groups of one (degree, column block) share
// its weights, so a degree stays on one XCD and its workgroups are neighbours in that XCD's queue, row groups fastest.
// Only row groups that exist are enumerated (a degree has (l + 1) B rows): XCD x serves the degrees L-1-x, L-9-x, ...
// (largest first: they have the most orders, hence the most rows) and a workgroup finds its place by walking that list.
__device__ __forceinline__ bool dh_map(const DhconvArgs& a, int group, int& l, int& ob, int& r0, int& ncols, int& rot) {
    int q = blockIdx.x >> 3;
    for (int lidx = blockIdx.x & 7; lidx < a.L; lidx += 8) {
        const int ll = a.L - 1 - lidx;
        const int nc_l = (a.tri ? min(ll + 1, a.M) : a.M) * a.B;      // rows (m, b) present at this degree
        const int t = (nc_l + group - 1) / group;
        const int n = a.nob * t;
        if (q < n) {
            l = ll;
            ob = q / t;
            const int rt = q - ob * t;
            r0 = rt * group;
            ncols = nc_l;
            rot = lidx + ob + rt;
            return true;
        }
        q -= n;
    }
    return false;
}

// number of workgroups dh_map enumerates: 8 x the longest XCD queue
static inline int64_t dh_blocks(const DhconvArgs& a, int group) {
    int64_t longest = 0;
    for (int x = 0; x < 8; ++x) {
        int64_t n = 0;
        for (int lidx = x; lidx < a.L; lidx += 8) {
            const int ll = a.L - 1 - lidx;
            const int64_t nc_l = (int64_t)(a.tri ? (ll + 1 < a.M ? ll + 1 : a.M) : a.M) * a.B;
            n += a.nob * ((nc_l + group - 1) / group);
        }
        longest = n > longest ? n : longest;
    }
    return 8 * longest;
}

}  // namespace sfno
