// permutedims when the source's first dim or the destination's first dim is short and a third dim can lengthen the
// runs: (2, N, 2) -> (2, N, 2) with perm (3, 2, 1), (4, 32, N) -> (N, 32, 4), (8, N, 8) -> (8, N, 8).  64 x 64 tiles over
// (source dim 1, destination dim 1) are almost empty there -- one workgroup per 4 elements in the first example.
//
// A workgroup moves a box X x Y x Z: X along the source's first dim (all of it when it is short), Z along the
// destination's first dim (all of it when it is short), Y a stretch of a third dim -- the source's second dim or the
// destination's second dim.  With X whole, the box's (x, y) planes are contiguous in the source; with Z whole, its
// (z, y) planes are contiguous in the destination.  The box is read in source order into LDS and written in
// destination order; each thread walks its elements with carried (x, y, z) counters instead of divisions.
// LDS holds element (x, y, z) at x + TX * y + zpitch * z with zpitch odd: the lanes of a store sweep z first.
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

constexpr int PERM_SLAB_MAX_DIMS = 8;
constexpr int PERM_SLAB_THREADS = 256;
constexpr int PERM_SLAB_SHORT = 64;        // a leading extent below this counts as short
constexpr int PERM_SLAB_LONG_CHUNK = 64;   // elements of a long leading dim in a box ...
constexpr int PERM_SLAB_LONG_MAX = 256;    // ... and when the third dim is used up and the budget is not

// Elements of LDS the kernel needs for a box budget of `budget` elements (zpitch rounds up to odd: at most TZ more).
constexpr int perm_slab_lds_elems(int budget) { return budget + PERM_SLAB_LONG_MAX; }

struct PermSlabGeom {
    int nd;                                 // merged dims
    int p, y;                               // merged source dim that leads the destination; the third dim of the box
    int64_t ext[PERM_SLAB_MAX_DIMS];
    int64_t sstride[PERM_SLAB_MAX_DIMS];
    int64_t dstride[PERM_SLAB_MAX_DIMS];
    int32_t TX, TY, TZ, zpitch;
    int64_t tilesx, tilesy, tilesz, blocks;
};

struct PermSlabBox {
    int64_t sbase, dbase;                   // offsets (elements) of the box's first element
    int32_t nx, ny, nz;                     // the box's actual extents (edges are ragged)
};

// Chooses the box; false when this mapping does not apply (then the tiles do the work).
inline bool perm_slab_geometry(const int64_t* ext_in, const int64_t* dstride_in, int nd, int p, int budget, PermSlabGeom* out) {
    if (nd < 2 || nd > PERM_SLAB_MAX_DIMS || p == 0) return false;
    // a plain transpose with a short side (17 x N <-> N x 17) is the same box with a third dim of extent 1
    int64_t ext[PERM_SLAB_MAX_DIMS + 1], dstride[PERM_SLAB_MAX_DIMS + 1];
    for (int d = 0; d < nd; ++d) { ext[d] = ext_in[d]; dstride[d] = dstride_in[d]; }
    if (nd == 2) { ext[2] = 1; dstride[2] = 0; nd = 3; }
    const int64_t a = ext[0], b = ext[p];
    const bool short_x = a < PERM_SLAB_SHORT, short_z = b < PERM_SLAB_SHORT;
    if (!short_x && !short_z) return false;
    // the destination's second dim: the merged source dim with the smallest destination stride above 1
    int q = -1;
    for (int d = 0; d < nd; ++d)
        if (d != p && (q < 0 || dstride[d] < dstride[q])) q = d;
    // the third dim: next to the short side (the shorter one when both are short)
    int y;
    const bool src_side = short_x && (!short_z || a <= b);
    if (src_side) y = (p != 1) ? 1 : (q != 0 ? q : -1);
    else y = (q != 0) ? q : (p != 1 ? 1 : -1);
    if (y < 0 || y == 0 || y == p) return false;
    PermSlabGeom g{};
    g.nd = nd;
    g.p = p;
    g.y = y;
    int64_t ss = 1;
    for (int d = 0; d < nd; ++d) {
        g.ext[d] = ext[d];
        g.sstride[d] = ss;
        g.dstride[d] = dstride[d];
        ss *= ext[d];
    }
    g.TX = (int32_t)(short_x ? a : (a < PERM_SLAB_LONG_CHUNK ? a : PERM_SLAB_LONG_CHUNK));
    g.TZ = (int32_t)(short_z ? b : (b < PERM_SLAB_LONG_CHUNK ? b : PERM_SLAB_LONG_CHUNK));
    int64_t ty = budget / ((int64_t)g.TX * g.TZ);
    if (ty < 1) return false;
    if (ty > ext[y]) ty = ext[y];
    g.TY = (int32_t)ty;
    if (ty == ext[y]) {
        // the third dim is used up: spend the rest of the budget on the long side
        int64_t room = budget / ((int64_t)(short_x ? g.TX : g.TZ) * g.TY);
        if (room > PERM_SLAB_LONG_MAX) room = PERM_SLAB_LONG_MAX;
        if (!short_x && room > g.TX) g.TX = (int32_t)(room < a ? room : a);
        if (!short_z && room > g.TZ) g.TZ = (int32_t)(room < b ? room : b);
    }
    g.zpitch = (g.TX * g.TY) | 1;
    g.tilesx = (a + g.TX - 1) / g.TX;
    g.tilesy = (ext[y] + g.TY - 1) / g.TY;
    g.tilesz = (b + g.TZ - 1) / g.TZ;
    int64_t blocks = g.tilesx * g.tilesy;            // small factors: no overflow before the checks below
    if (blocks > 0x7fffffff / g.tilesz) return false;
    blocks *= g.tilesz;
    for (int d = 1; d < nd; ++d) {
        if (d == p || d == y) continue;
        if (blocks > 0x7fffffff / ext[d]) return false;
        blocks *= ext[d];
    }
    g.blocks = blocks;
    *out = g;
    return true;
}

RK_HD PermSlabBox perm_slab_box(const PermSlabGeom& g, int64_t block) {
    int64_t b = block;
    const int64_t tx = b % g.tilesx; b /= g.tilesx;
    const int64_t ty = b % g.tilesy; b /= g.tilesy;
    const int64_t tz = b % g.tilesz; b /= g.tilesz;
    const int64_t x0 = tx * g.TX, y0 = ty * g.TY, z0 = tz * g.TZ;
    PermSlabBox box;
    box.sbase = x0 + y0 * g.sstride[g.y] + z0 * g.sstride[g.p];
    box.dbase = z0 + y0 * g.dstride[g.y] + x0 * g.dstride[0];
    for (int d = 1; d < g.nd; ++d) {
        if (d == g.p || d == g.y) continue;
        const int64_t c = b % g.ext[d];
        b /= g.ext[d];
        box.sbase += c * g.sstride[d];
        box.dbase += c * g.dstride[d];
    }
    const int64_t rx = g.ext[0] - x0, ry = g.ext[g.y] - y0, rz = g.ext[g.p] - z0;
    box.nx = (int32_t)(rx < g.TX ? rx : g.TX);
    box.ny = (int32_t)(ry < g.TY ? ry : g.TY);
    box.nz = (int32_t)(rz < g.TZ ? rz : g.TZ);
    return box;
}

// Three nested counters (fastest n0, then n1, then the rest) that advance by PERM_SLAB_THREADS elements a step.
struct PermSlabWalk {
    int32_t c0, c1, c2;            // position
    int32_t s0, s1, s2;            // the step, decomposed
    int32_t n0, n1;
    RK_HD void start(int32_t t, int32_t n0_, int32_t n1_) {
        n0 = n0_; n1 = n1_;
        c0 = t % n0;
        int32_t r = t / n0;
        c1 = r % n1;
        c2 = r / n1;
        s0 = PERM_SLAB_THREADS % n0;
        r = PERM_SLAB_THREADS / n0;
        s1 = r % n1;
        s2 = r / n1;
    }
    RK_HD void next() {
        c0 += s0;
        int32_t carry = c0 >= n0 ? 1 : 0;
        c0 -= carry ? n0 : 0;
        c1 += s1 + carry;                  // < 2 * n1
        carry = c1 >= n1 ? 1 : 0;
        c1 -= carry ? n1 : 0;
        c2 += s2 + carry;
    }
};

// Thread t of the box: copies its share of the source into LDS (source order: x fastest).  Four elements a round:
// their loads are issued together (one for 16-byte elements: the compiler keeps a round of those in private memory).
template <typename T> struct PermSlabRound { static constexpr int N = sizeof(T) >= 16 ? 1 : 4; };

template <typename T>
RK_HD void perm_slab_load(const PermSlabGeom& g, const PermSlabBox& box, int32_t t, const T* src, T* lds) {
    const int64_t ssy = g.sstride[g.y], ssz = g.sstride[g.p];
    PermSlabWalk w;
    w.start(t, box.nx, box.ny);
    while (w.c2 < box.nz) {
        constexpr int U = PermSlabRound<T>::N;
        T v[U];
        int32_t at[U];
        bool live[U];
#ifdef __HIPCC__
#pragma unroll
#endif
        for (int u = 0; u < U; ++u) {
            live[u] = w.c2 < box.nz;
            at[u] = w.c0 + g.TX * w.c1 + g.zpitch * w.c2;
            if (live[u]) v[u] = src[box.sbase + w.c0 + w.c1 * ssy + w.c2 * ssz];
            w.next();
        }
#ifdef __HIPCC__
#pragma unroll
#endif
        for (int u = 0; u < U; ++u)
            if (live[u]) lds[at[u]] = v[u];
    }
}

// Thread t of the box: writes its share of LDS to the destination (destination order: z fastest).
template <typename T>
RK_HD void perm_slab_store(const PermSlabGeom& g, const PermSlabBox& box, int32_t t, const T* lds, T* dst) {
    const int64_t dsy = g.dstride[g.y], dsx = g.dstride[0];
    PermSlabWalk w;
    w.start(t, box.nz, box.ny);
    while (w.c2 < box.nx) {
        constexpr int U = PermSlabRound<T>::N;
        T v[U];
        int64_t at[U];
        bool live[U];
#ifdef __HIPCC__
#pragma unroll
#endif
        for (int u = 0; u < U; ++u) {
            live[u] = w.c2 < box.nx;
            at[u] = box.dbase + w.c0 + w.c1 * dsy + w.c2 * dsx;
            if (live[u]) v[u] = lds[w.c2 + g.TX * w.c1 + g.zpitch * w.c0];
            w.next();
        }
#ifdef __HIPCC__
#pragma unroll
#endif
        for (int u = 0; u < U; ++u)
            if (live[u]) dst[at[u]] = v[u];
    }
}

// ---- the same two steps with 16-byte global accesses ---------------------------------------------------------------------
// With the source's whole first dim in the box and the box's third dim next to it, a z plane of the box is one
// contiguous run of nx * ny elements; with the destination's whole first dim in the box and the third dim next to it
// there, every x of the box is one contiguous run of nz * ny elements in the destination.  When such runs start at
// multiples of 16 bytes and hold whole 16-byte vectors, a thread moves a vector at a time between global memory and
// registers (LDS is still accessed by element: its layout keeps the odd pitch).  Four bytes a lane keep too few
// bytes in flight: (2, N, 2) -> perm (3, 2, 1) Float32 ran at 3.1 TB/s.
// `ldv(offset, out)` reads V elements at `offset` of the source, `stv(offset, in)` writes V elements of the destination.
template <typename T> struct PermSlabVec { static constexpr int V = sizeof(T) < 16 ? 16 / (int)sizeof(T) : 1; };

template <typename T>
RK_HD bool perm_slab_load_vec_ok(const PermSlabGeom& g, const PermSlabBox& box, const void* src) {
    constexpr int V = PermSlabVec<T>::V;
    return V > 1 && box.nx == g.ext[0] && g.sstride[g.y] == g.ext[0] && (box.nx * box.ny) % V == 0 && box.sbase % V == 0 &&
           (box.nz == 1 || g.sstride[g.p] % V == 0) && ((uintptr_t)src & 15) == 0;
}
template <typename T>
RK_HD bool perm_slab_store_vec_ok(const PermSlabGeom& g, const PermSlabBox& box, const void* dst) {
    constexpr int V = PermSlabVec<T>::V;
    return V > 1 && box.nz == g.ext[g.p] && g.dstride[g.y] == g.ext[g.p] && (box.nz * box.ny) % V == 0 && box.dbase % V == 0 &&
           (box.nx == 1 || g.dstride[0] % V == 0) && ((uintptr_t)dst & 15) == 0;
}

template <typename T, typename LoadVec, typename Lds>
RK_HD void perm_slab_load_vec(const PermSlabGeom& g, const PermSlabBox& box, int32_t t, LoadVec&& ldv, Lds&& lds) {
    constexpr int V = PermSlabVec<T>::V, U = 4;
    const int32_t per_plane = box.nx * box.ny / V, total = per_plane * box.nz;
    const int64_t ssz = g.sstride[g.p];
    for (int32_t v0 = t; v0 < total; v0 += U * PERM_SLAB_THREADS) {
        T val[U][V];
        int32_t at[U];
#ifdef __HIPCC__
#pragma unroll
#endif
        for (int u = 0; u < U; ++u) {
            const int32_t v = v0 + u * PERM_SLAB_THREADS;
            at[u] = -1;
            if (v < total) {
                const int32_t z = v / per_plane, r = v - z * per_plane;
                at[u] = r * V + g.zpitch * z;                       // x + TX * y = position in the plane, TX = nx
                ldv(box.sbase + (int64_t)z * ssz + (int64_t)r * V, val[u]);
            }
        }
#ifdef __HIPCC__
#pragma unroll
#endif
        for (int u = 0; u < U; ++u) {
            if (at[u] >= 0) {
#ifdef __HIPCC__
#pragma unroll
#endif
                for (int j = 0; j < V; ++j) lds[at[u] + j] = val[u][j];
            }
        }
    }
}

template <typename T, typename Lds, typename StoreVec>
RK_HD void perm_slab_store_vec(const PermSlabGeom& g, const PermSlabBox& box, int32_t t, Lds&& lds, StoreVec&& stv) {
    constexpr int V = PermSlabVec<T>::V;
    const int32_t per_x = box.nz * box.ny / V, total = per_x * box.nx;
    const int64_t dsx = g.dstride[0];
    for (int32_t v = t; v < total; v += PERM_SLAB_THREADS) {
        const int32_t x = v / per_x, r = v - x * per_x;
        const int32_t f0 = r * V;
        int32_t y = f0 / box.nz, z = f0 - y * box.nz;
        T val[V];
#ifdef __HIPCC__
#pragma unroll
#endif
        for (int j = 0; j < V; ++j) {
            val[j] = lds[x + g.TX * y + g.zpitch * z];
            ++z;
            if (z == box.nz) { z = 0; ++y; }
        }
        stv(box.dbase + (int64_t)x * dsx + f0, val);
    }
}

}  // namespace rk
