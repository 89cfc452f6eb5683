// permutedims when the source's or the destination's contiguous dim is short (at most PERM_SMALL_MAX elements): the
// (N, 3) <-> (3, N) and (N, 4) <-> (4, N) conversions between arrays of structures and structures of arrays, batches of
// tiny matrices.  64 x 64 tiles through LDS leave most of every tile empty there.  Here a lane owns one run of the short
// dim: it reads the run's elements (stride 1 when the short dim is the source's first, else the source stride of that
// dim) and writes them (the destination stride of that dim, 1 when it is the destination's first).  Lanes advance along
// the long dim that is contiguous on the other side, so every load (or store) instruction of a wave covers consecutive
// addresses, and the runs of neighbouring lanes are neighbours in memory on the short side.
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
    int nd;                            // looped dims: every merged dim except the short one, the lane dim first
    int64_t ext[PERM_MAX_DIMS];
    int64_t sstride[PERM_MAX_DIMS];    // source / destination strides (elements) of the looped dims
    int64_t dstride[PERM_MAX_DIMS];
    int32_t small;                     // extent of the short dim
    int64_t small_sstride, small_dstride;
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
// merged source dim that is contiguous in the destination (p != 0).  Returns false when neither side is short.
inline bool perm_small_geometry(const int64_t* ext, const int64_t* dstride, int nd, int p, int64_t total, PermSmallGeom* out) {
    if (nd < 2 || nd > PERM_MAX_DIMS || p <= 0 || p >= nd) return false;
    int64_t sstr[PERM_MAX_DIMS];
    int64_t s = 1;
    for (int d = 0; d < nd; ++d) { sstr[d] = s; s *= ext[d]; }
    int small_dim, lane_dim;
    // prefer the short destination run (its stores become one contiguous piece per lane); else the short source run
    // and only when the runs of neighbouring lanes are neighbours in memory on the short side (the lane dim follows the
    // short dim directly there); otherwise every access of a run is a scattered 4- or 8-byte piece
    // ((1048576, 2, 8) -> (8, 2, 1048576): 145 us this way, 62 us with tiles)
    if (ext[p] <= PERM_SMALL_MAX && dstride[0] == ext[p]) { small_dim = p; lane_dim = 0; }
    else if (ext[0] <= PERM_SMALL_MAX && p == 1) { small_dim = 0; lane_dim = p; }
    else return false;
    PermSmallGeom g{};
    g.small = (int32_t)ext[small_dim];
    g.small_sstride = sstr[small_dim];
    g.small_dstride = dstride[small_dim];
    g.n_threads = total / ext[small_dim];
    int k = 0;
    g.ext[k] = ext[lane_dim]; g.sstride[k] = sstr[lane_dim]; g.dstride[k] = dstride[lane_dim]; ++k;
    for (int d = 0; d < nd; ++d) {
        if (d == small_dim || d == lane_dim) continue;
        g.ext[k] = ext[d]; g.sstride[k] = sstr[d]; g.dstride[k] = dstride[d]; ++k;
    }
    g.nd = k;
    *out = g;
    return true;
}

}  // namespace rk
