// permutedims when a short block of dims leads the source or the destination (at most PERM_SMALL_MAX elements): the
// (N, 3) <-> (3, N) and (N, 4) <-> (4, N) conversions between arrays of structures and structures of arrays,
// (2, 3, N) <-> (N, 3, 2), batches of tiny matrices.  64 x 64 tiles through LDS leave most of every tile empty there.
// Here a lane owns one run = one instance of the short block: contiguous on the side the block leads, scattered by the
// other side's strides.  Lanes advance along the long dim that is contiguous on the other side, so every load (or
// store) instruction of a wave covers consecutive addresses, and the runs of neighbouring lanes are neighbours in
// memory on the run's contiguous side.
//
// The index mapping is host-callable: a brute-force check over every thread of many shapes runs on the CPU.
#pragma once
#include <cstdint>

#ifndef RK_HD
#ifdef __HIPCC__
#define RK_HD __host__ __device__ __forceinline__
#else
#define RK_HD inline
#endif
#endif

namespace rk {

constexpr int PERM_SMALL_MAX = 16;
constexpr int PERM_MAX_DIMS = 8;

struct PermSmallGeom {
    int64_t n_threads;                 // runs = elements / small
    int nd;                            // looped dims: every merged dim outside the short block, the lane dim first
    int64_t ext[PERM_MAX_DIMS];
    int64_t sstride[PERM_MAX_DIMS];    // source / destination strides (elements) of the looped dims
    int64_t dstride[PERM_MAX_DIMS];
    int32_t small;                     // elements of a run (the product of the short block's extents)
    int64_t run_soff[PERM_SMALL_MAX];  // source / destination offset of element j of a run; one of the two is j
    int64_t run_doff[PERM_SMALL_MAX];
};

// Source and destination offsets (elements) of the first element of run `idx`.
RK_HD void perm_small_offsets(const PermSmallGeom& g, int64_t idx, int64_t* soff, int64_t* doff) {
    int64_t rem = idx, s = 0, d = 0;
    for (int k = 0; k < g.nd; ++k) {
        int64_t c;
        if (k == g.nd - 1) c = rem;
        else { const int64_t q = rem / g.ext[k]; c = rem - q * g.ext[k]; rem = q; }
        s += c * g.sstride[k];
        d += c * g.dstride[k];
    }
    *soff = s;
    *doff = d;
}

// Geometry from merged source extents `ext[0..nd)`, the destination stride of every merged source dim, and p = the
// merged source dim that is contiguous in the destination (p != 0).  Two shapes qualify:
//   * the source's leading dims 0 .. p-1 hold at most max_run elements together (2 x 3 x N -> N x 3 x 2, 3 x N -> N x 3):
//     a run is that block, contiguous in the source, its elements scattered by the destination strides; lanes along p;
//   * the destination's leading dims, up to the one that is the source's dim 0, hold at most max_run elements
//     (N x 3 x 2 -> 2 x 3 x N, N x 4 -> 4 x N): a run is contiguous in the destination, gathered by source strides;
//     lanes along dim 0.
// In both the runs of neighbouring lanes are neighbours in memory on the run's contiguous side.  Returns false otherwise.
inline bool perm_small_geometry(const int64_t* ext, const int64_t* dstride, int nd, int p, int64_t total, int max_run, PermSmallGeom* out) {
    if (nd < 2 || nd > PERM_MAX_DIMS || p <= 0 || p >= nd || max_run > PERM_SMALL_MAX) return false;
    int64_t sstr[PERM_MAX_DIMS];
    int64_t s = 1;
    for (int d = 0; d < nd; ++d) { sstr[d] = s; s *= ext[d]; }
    bool in_block[PERM_MAX_DIMS] = {};
    int block[PERM_MAX_DIMS], nb = 0;      // dims of the short block, fastest first on the run's contiguous side
    int lane_dim = -1;
    bool src_run = false;
    // destination order of the merged source dims: increasing dstride
    int dorder[PERM_MAX_DIMS];
    for (int d = 0; d < nd; ++d) dorder[d] = d;
    for (int i = 1; i < nd; ++i)
        for (int j = i; j > 0 && dstride[dorder[j]] < dstride[dorder[j - 1]]; --j) { const int t = dorder[j]; dorder[j] = dorder[j - 1]; dorder[j - 1] = t; }
    {   // destination-leading block: dorder[0] = p, ..., until source dim 0 appears
        int64_t prod = 1;
        int k = 0;
        while (k < nd && dorder[k] != 0) { prod *= ext[dorder[k]]; ++k; }
        if (k >= 1 && k < nd && prod <= max_run) {
            for (int i = 0; i < k; ++i) { block[nb++] = dorder[i]; in_block[dorder[i]] = true; }
            lane_dim = 0;
        }
    }
    if (lane_dim < 0) {   // source-leading block: dims 0 .. p-1
        int64_t prod = 1;
        for (int d = 0; d < p; ++d) prod *= ext[d];
        if (prod <= max_run) {
            for (int d = 0; d < p; ++d) { block[nb++] = d; in_block[d] = true; }
            lane_dim = p;
            src_run = true;
        }
    }
    if (lane_dim < 0) return false;
    PermSmallGeom g{};
    int64_t run = 1;
    for (int i = 0; i < nb; ++i) run *= ext[block[i]];
    g.small = (int32_t)run;
    for (int64_t j = 0; j < run; ++j) {    // coordinates of element j inside the block, the first block dim fastest
        int64_t rem = j, so = 0, dof = 0;
        for (int i = 0; i < nb; ++i) {
            const int64_t c = rem % ext[block[i]];
            rem /= ext[block[i]];
            so += c * sstr[block[i]];
            dof += c * dstride[block[i]];
        }
        g.run_soff[j] = so;
        g.run_doff[j] = dof;
    }
    (void)src_run;
    g.n_threads = total / run;
    int k = 0;
    g.ext[k] = ext[lane_dim]; g.sstride[k] = sstr[lane_dim]; g.dstride[k] = dstride[lane_dim]; ++k;
    for (int d = 0; d < nd; ++d) {
        if (in_block[d] || d == lane_dim) continue;
        g.ext[k] = ext[d]; g.sstride[k] = sstr[d]; g.dstride[k] = dstride[d]; ++k;
    }
    g.nd = k;
    *out = g;
    return true;
}

}  // namespace rk
