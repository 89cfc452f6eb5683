// permutedims(src, perm) / permutedims!(dst, src, perm) for dense column-major arrays of any element size.
// The reference takes this from GPUArrays (one element per work-item, dest[I_perm] = src[I]; benchmarked in
// perf/array.jl:151-155); here:
//   * dims that stay neighbours in the same order are merged, extents of 1 dropped;
//   * if the first dim stays first, rows move whole: 16-byte units (or elements), coalesced on both sides;
//   * if the leading dims of the source (up to the one that becomes the destination's first) or of the destination
//     (up to the source's first) hold at most 8 elements -- (N, 3) <-> (3, N), (2, 3, N) <-> (N, 3, 2), batches of
//     tiny matrices -- a lane moves one such run (rk_permute_small.hpp);
//   * if the source's or the destination's first dim is short (< 64) and a third dim can lengthen the runs --
//     (2, N, 2) with perm (3, 2, 1), (4, 32, N) -> (N, 32, 4) -- a workgroup moves a box of three dims through LDS
//     (rk_permute_slab.hpp);
//   * otherwise 64 x 64 tiles over (src dim 1, the src dim that becomes dst dim 1) go through LDS, so that loads
//     run along the source's contiguous axis and stores along the destination's.
// 2 x elsize bytes per element, no workspace.
#include "rk_common.hpp"
#include "rk_permute_small.hpp"
#include "rk_permute_slab.hpp"

namespace rk {

struct PermGeom {
    int64_t ext[RK_MAX_DIMS];       // merged src extents
    int64_t dstride[RK_MAX_DIMS];   // dst stride (elements) of merged src dim d
    int64_t total;                  // elements
    int nd;
    int p;                          // merged src dim that is contiguous in dst
};

typedef uint32_t pu32x4 __attribute__((ext_vector_type(4)));
template <int E> struct PElem;
template <> struct PElem<1> { typedef uint8_t type; };
template <> struct PElem<2> { typedef uint16_t type; };
template <> struct PElem<4> { typedef uint32_t type; };
template <> struct PElem<8> { typedef uint64_t type; };
template <> struct PElem<16> { struct type { uint64_t lo, hi; }; };

// First dim stays first: unit i of src (dim 0 counted in units) goes to the offset given by the dst strides.
template <typename UNIT, typename I>
__global__ __launch_bounds__(256) void permute_rows_kernel(const UNIT* __restrict__ src, UNIT* __restrict__ dst, PermGeom g) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= g.total) return;
    I rem = (I)i;
    int64_t o = 0;
    for (int d = 0; d < g.nd; ++d) {
        const I e = (I)g.ext[d];
        I c;
        if (d == g.nd - 1) c = rem;
        else { const I q = rem / e; c = rem - q * e; rem = q; }
        o += (int64_t)c * g.dstride[d];
    }
    dst[o] = src[i];
}

// grid.x enumerates (tile along src dim 0, tile along src dim p, every other dim), the tile pairs in diagonal order:
// workgroups that run together then differ in both tile coordinates, so neither their loads nor their stores sit a
// power-of-two pitch apart (8192 x 8192 Float32 transpose: 3.8 -> 5.7 TB/s).  PT = tile edge (64; 32 for
// 16-byte elements, to fit the tile in LDS); the 256 threads form 256 / PT rows of PT lanes: a load reads PT
// consecutive elements of src dim 0, a store writes PT consecutive elements of dst dim 0 (= src dim p).  The LDS
// tile is padded by one column: column reads hit distinct banks.
template <typename T, int PT>
__global__ __launch_bounds__(256) void permute_tiles_kernel(const T* __restrict__ src, T* __restrict__ dst, PermGeom g, int64_t tiles0,
                                                            int64_t tilesp) {
    __shared__ T tile[PT][PT + 1];
    constexpr int NY = 256 / PT;
    const int lane = threadIdx.x % PT, wave = threadIdx.x / PT;
    int64_t b = blockIdx.x;
    const int64_t t0 = b % tiles0; b /= tiles0;
    const int64_t tp = (b % tilesp + t0) % tilesp; b /= tilesp;      // diagonal order
    int64_t sbase = 0, dbase = 0, sstride = 1, sstride_p = 0;
    for (int d = 0; d < g.nd; ++d) {
        if (d == g.p) sstride_p = sstride;
        else if (d != 0) {
            const int64_t c = b % g.ext[d];
            b /= g.ext[d];
            sbase += c * sstride;
            dbase += c * g.dstride[d];
        }
        sstride *= g.ext[d];
    }
    const int64_t i0 = t0 * PT, p0 = tp * PT;
    const int64_t n0 = g.ext[0], np = g.ext[g.p];
    if (i0 + lane < n0) {
        const T* s = src + sbase + i0 + lane;
#pragma unroll 4
        for (int j = wave; j < PT; j += NY)
            if (p0 + j < np) tile[j][lane] = s[(p0 + j) * sstride_p];
    }
    __syncthreads();
    if (p0 + lane < np) {
        T* q = dst + dbase + p0 + lane;
        const int64_t ds0 = g.dstride[0];
#pragma unroll 4
        for (int j = wave; j < PT; j += NY)
            if (i0 + j < n0) q[(i0 + j) * ds0] = tile[lane][j];
    }
}

// The same tiling with 16-byte accesses on both sides (V = 16 / sizeof(T) elements per lane): TE / V lanes cover a
// tile row, so a request still spans TE * sizeof(T) contiguous bytes but with a quarter (or less) of the
// instructions.  Needs ext[0] % V == 0 and ext[p] % V == 0 and 16-byte aligned arrays: every vector is then
// entirely inside or outside the array, and every row start is aligned.
// ELEMS (4- and 8-byte elements): extents and addresses need not be whole vectors -- global memory takes 16-byte
// accesses at any element-aligned address.  The last vector of a row starts V elements before the row's end instead of
// running past it; where that reaches back into the tile in front, the elements of this tile go one by one.
constexpr int PERM_XCDS = 8;
template <typename T, int TE, bool ELEMS>
__global__ __launch_bounds__(256) void permute_tiles_vec_kernel(const T* __restrict__ src, T* __restrict__ dst, PermGeom g, int64_t tiles0,
                                                                int64_t tilesp, int by_xcd) {
    constexpr int V = 16 / sizeof(T), LR = TE / V, RP = 256 / LR;
    typedef typename VecOf<T, V>::type VT;
    __shared__ T tile[TE][TE + 1];
    const int c = threadIdx.x % LR, r = threadIdx.x / LR;
    // Workgroups go round-robin to the 8 XCDs, each with an L2 of its own.  A tile row of the destination is TE
    // elements; unless the destination's rows are whole 128-byte lines, two tiles that are neighbours along p write
    // parts of one line, and from different L2s -- or from one, long apart -- those are two partial write-backs
    // (5000 x 6001 Float32: 2.5 TB/s against 4.0 for 5000 x 6000).  by_xcd: every XCD takes a contiguous eighth of the
    // tile rows tp and walks it along p first, so neighbours along p follow each other in one L2: 5000 x 6001 95 -> 65 us,
    // and whole-line rows gain too (8000 x 8000 102 -> 92, 5000 x 6000 60 -> 48).  Dealing tile COLUMNS to the XCDs
    // (p-neighbours ten launches apart) gave 79 us, bands walked along dim 0 first 90.  Pitches that are multiples of
    // 4 KiB keep the plain diagonal order (consecutive tiles must not hit one channel; 8192 x 8192: 94 us, bands 98).
    int64_t b = blockIdx.x;
    int64_t t0, tp;
    if (by_xcd == 2) {
        // fewer than seven tile rows, no bands to hand out: every XCD takes each eighth tile COLUMN and walks it along p, so the
        // few neighbours along p are consecutive workgroups of one L2 (90 001 x 333 Float32: 100 -> 85 us, Float64 150 -> 133)
        const int64_t xcd = b % PERM_XCDS; b /= PERM_XCDS;
        const int64_t cols = (tiles0 + PERM_XCDS - 1) / PERM_XCDS;
        tp = b % tilesp; b /= tilesp;
        t0 = (b % cols) * PERM_XCDS + xcd; b /= cols;
        if (t0 >= tiles0) return;
    } else if (by_xcd) {
        const int64_t xcd = b % PERM_XCDS; b /= PERM_XCDS;
        const int64_t rows = (tilesp + PERM_XCDS - 1) / PERM_XCDS;   // tile rows per XCD
        tp = xcd * rows + b % rows; b /= rows;                       // along p first: the neighbours follow each other
        t0 = b % tiles0; b /= tiles0;
        if (tp >= tilesp) return;                                    // the last band is short: whole workgroups
    } else {
        t0 = b % tiles0; b /= tiles0;
        tp = (b % tilesp + t0) % tilesp; b /= tilesp;                // diagonal order
    }
    int64_t sbase = 0, dbase = 0, sstride = 1, sstride_p = 0;
    for (int d = 0; d < g.nd; ++d) {
        if (d == g.p) sstride_p = sstride;
        else if (d != 0) {
            const int64_t cd = b % g.ext[d];
            b /= g.ext[d];
            sbase += cd * sstride;
            dbase += cd * g.dstride[d];
        }
        sstride *= g.ext[d];
    }
    const int64_t i0 = t0 * TE, p0 = tp * TE;
    const int64_t n0 = g.ext[0], np = g.ext[g.p];
    if (i0 + c * V < n0) {
        // first column of this lane's vector, relative to the tile: negative when the row's last vector reaches back
        const int lc = (ELEMS && i0 + c * V + V > n0) ? (int)(n0 - V - i0) : c * V;
        const T* s = src + sbase + i0 + lc;
#pragma unroll
        for (int j = r; j < TE; j += RP) {
            if (p0 + j < np) {
                VT v;
                if constexpr (ELEMS) v = load_nt_elems<T, V>(s + (p0 + j) * sstride_p);
                else v = load_nt((const VT*)(s + (p0 + j) * sstride_p));
#pragma unroll
                for (int k = 0; k < V; ++k)
                    if (!ELEMS || lc + k >= 0) tile[j][lc + k] = v[k];
            }
        }
    }
    __syncthreads();
    if (p0 + c * V < np) {
        const int lp = (ELEMS && p0 + c * V + V > np) ? (int)(np - V - p0) : c * V;
        T* q = dst + dbase + p0 + lp;
        const int64_t ds0 = g.dstride[0];
#pragma unroll
        for (int j = r; j < TE; j += RP) {
            if (i0 + j < n0) {
                VT v;
#pragma unroll
                for (int k = 0; k < V; ++k) v[k] = tile[(ELEMS && lp + k < 0) ? 0 : lp + k][j];
                if constexpr (ELEMS) {
                    if (lp >= 0) store_nt_elems<T, V>(q + (i0 + j) * ds0, v);
                    else {
#pragma unroll
                        for (int k = 0; k < V; ++k)
                            if (lp + k >= 0) q[(i0 + j) * ds0 + k] = v[k];
                    }
                } else store_nt((VT*)(q + (i0 + j) * ds0), v);
            }
        }
    }
}

// One run of the short dim per lane (geometry and index mapping: rk_permute_small.hpp).
template <typename T>
__global__ __launch_bounds__(256) void permute_small_kernel(const T* __restrict__ src, T* __restrict__ dst, PermSmallGeom g) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= g.n_threads) return;
    int64_t so, dofs;
    perm_small_offsets(g, idx, &so, &dofs);
    T v[PERM_SMALL_MAX];
#pragma unroll
    for (int j = 0; j < PERM_SMALL_MAX; ++j)
        if (j < g.small) v[j] = src[so + g.run_soff[j]];
#pragma unroll
    for (int j = 0; j < PERM_SMALL_MAX; ++j)
        if (j < g.small) dst[dofs + g.run_doff[j]] = v[j];
}

// A box of three dims through LDS: read in source order, written in destination order.
template <typename T, int BUDGET>
__global__ __launch_bounds__(PERM_SLAB_THREADS) void permute_slab_kernel(const T* __restrict__ src, T* __restrict__ dst, PermSlabGeom g) {
    __shared__ T lds[perm_slab_lds_elems(BUDGET)];
    const PermSlabBox box = perm_slab_box(g, (int64_t)blockIdx.x);
    constexpr int V = PermSlabVec<T>::V;
    struct alignas(16) Vec { T e[V]; };
    if (perm_slab_load_vec_ok<T>(g, box, src)) {
        perm_slab_load_vec<T>(g, box, (int32_t)threadIdx.x, [&](int64_t off, T (&out)[V]) {
            const Vec v = *(const Vec*)(src + off);
#pragma unroll
            for (int j = 0; j < V; ++j) out[j] = v.e[j];
        }, lds);
    } else {
        perm_slab_load(g, box, (int32_t)threadIdx.x, src, lds);
    }
    __syncthreads();
    if (perm_slab_store_vec_ok<T>(g, box, dst)) {
        perm_slab_store_vec<T>(g, box, (int32_t)threadIdx.x, lds, [&](int64_t off, const T (&in)[V]) {
            Vec v;
#pragma unroll
            for (int j = 0; j < V; ++j) v.e[j] = in[j];
            *(Vec*)(dst + off) = v;
        });
    } else {
        perm_slab_store(g, box, (int32_t)threadIdx.x, lds, dst);
    }
}

// ---- batches of small matrices: permutedims(A, (2, 1, 3)) of a 100 x 100 x N array ------------------------------
// 64 x 64 tiles over a 100 x 100 matrix are 61 % full (2.5 TB/s).  A matrix of up to 48 KiB is one contiguous run in
// the source and in the destination: a workgroup reads it whole with 16-byte loads (at element-aligned addresses, four
// in flight a lane), keeps it in LDS row by row with an odd pitch, and writes it whole in the destination's order.
// The LDS side is element by element with 4-way bank conflicts -- a twentieth of the workgroup's memory time.
template <typename T> struct PermMat { static constexpr int BUDGET = 49152 / (int)sizeof(T); };

template <typename T>
__global__ __launch_bounds__(256) void permute_matrices_kernel(const T* __restrict__ src, T* __restrict__ dst, int n0, int n1, int pitch) {
    constexpr int V = 16 / sizeof(T);
    typedef typename VecOf<T, V>::type VT;
    __shared__ T lds[PermMat<T>::BUDGET];
    const int M = n0 * n1, nv = M / V;
    const T* s = src + (int64_t)blockIdx.x * M;
    T* q = dst + (int64_t)blockIdx.x * M;
    const int t = threadIdx.x;
    // source order: element idx = i + n0 * j goes to lds[j * pitch + i]
    for (int v0 = 0; v0 < nv; v0 += 4 * 256) {
        VT x[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int v = v0 + u * 256 + t;
            x[u] = load_nt_elems<T, V>(s + (int64_t)(v < nv ? v : nv - 1) * V);      // unconditional: past the end, the last vector again
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int v = v0 + u * 256 + t;
            if (v < nv) {
                int j = (v * V) / n0, i = v * V - j * n0;
#pragma unroll
                for (int k = 0; k < V; ++k) {
                    lds[j * pitch + i] = x[u][k];
                    if (++i == n0) { i = 0; ++j; }
                }
            }
        }
    }
    for (int idx = nv * V + t; idx < M; idx += 256) { const int j = idx / n0; lds[j * pitch + idx - j * n0] = s[idx]; }
    __syncthreads();
    // destination order: element e = j + n1 * i comes from lds[j * pitch + i]
    for (int v = t; v < nv; v += 256) {
        int i = (v * V) / n1, j = v * V - i * n1;
        VT o;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            o[k] = lds[j * pitch + i];
            if (++j == n1) { j = 0; ++i; }
        }
        store_nt_elems<T, V>(q + (int64_t)v * V, o);
    }
    for (int e = nv * V + t; e < M; e += 256) { const int i = e / n1; q[e] = lds[(e - i * n1) * pitch + i]; }
}

template <int E>
static int32_t permute_elsize(const void* src, void* dst, PermGeom g, hipStream_t stream) {
    typedef typename PElem<E>::type T;
    if (g.p == 0) {
        // rows move whole; in 16-byte units when rows and every dst stride are whole units
        bool vector = is_aligned(src, 16) && is_aligned(dst, 16) && (g.ext[0] * E) % 16 == 0;
        PermGeom u = g;
        if (vector && E < 16) {
            const int per = 16 / E;
            u.ext[0] = g.ext[0] / per;
            u.total = g.total / per;
            for (int d = 1; d < g.nd; ++d) u.dstride[d] = g.dstride[d] / per;   // multiples of ext[0]
        }
        const int64_t blocks = (u.total + 255) / 256;
        if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
        const bool small = u.total <= 0xffffffffll;
        if (vector) {
            if (small) permute_rows_kernel<pu32x4, uint32_t><<<(unsigned)blocks, 256, 0, stream>>>((const pu32x4*)src, (pu32x4*)dst, u);
            else permute_rows_kernel<pu32x4, uint64_t><<<(unsigned)blocks, 256, 0, stream>>>((const pu32x4*)src, (pu32x4*)dst, u);
        } else {
            if (small) permute_rows_kernel<T, uint32_t><<<(unsigned)blocks, 256, 0, stream>>>((const T*)src, (T*)dst, u);
            else permute_rows_kernel<T, uint64_t><<<(unsigned)blocks, 256, 0, stream>>>((const T*)src, (T*)dst, u);
        }
        RK_LAUNCH_CHECK();
        return RK_SUCCESS;
    }
    if constexpr (E <= 8) {
        // a short contiguous dim on either side: tiles would be mostly empty
        // ((4194304, 3) -> (3, 4194304) Float32: 0.68 TB/s with tiles)
        PermSmallGeom sg;
        if (perm_small_geometry(g.ext, g.dstride, g.nd, g.p, g.total, 8, &sg)) {
            const int64_t blocks = (sg.n_threads + 255) / 256;
            if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
            permute_small_kernel<T><<<(unsigned)blocks, 256, 0, stream>>>((const T*)src, (T*)dst, sg);
            RK_LAUNCH_CHECK();
            return RK_SUCCESS;
        }
    }
    {
        // a short first dim on either side with a third dim to lengthen the runs: tiles over the two first dims alone
        // would be mostly empty ((2, 8388608, 2) -> perm (3, 2, 1) Float32: 17.9 ms with tiles, a workgroup per 4 elements)
        constexpr int BUDGET = 16384 / E;
        PermSlabGeom sl;
        if (perm_slab_geometry(g.ext, g.dstride, g.nd, g.p, BUDGET, &sl)) {
            permute_slab_kernel<T, BUDGET><<<(unsigned)sl.blocks, PERM_SLAB_THREADS, 0, stream>>>((const T*)src, (T*)dst, sl);
            RK_LAUNCH_CHECK();
            return RK_SUCCESS;
        }
    }
    if constexpr (E == 4 || E == 8) {
        // batches of matrices that the 64 x 64 tiles would fill to less than 80 %, whole matrices through LDS
        if (g.nd >= 2 && g.p == 1 && g.dstride[0] == g.ext[1] && g.ext[0] >= 16 / E && g.ext[1] >= 16 / E) {
            const int64_t n0 = g.ext[0], n1 = g.ext[1], M = n0 * n1, pitch = n0 | 1;
            bool batch_in_place = true;                      // the dims above the matrix keep their strides
            int64_t stride = M;
            for (int d = 2; d < g.nd; ++d) { batch_in_place = batch_in_place && g.dstride[d] == stride; stride *= g.ext[d]; }
            const int64_t nmat = g.total / M;
            const int64_t tiled = ((n0 + 63) / 64) * ((n1 + 63) / 64) * 4096;
            if (batch_in_place && n1 * pitch <= PermMat<T>::BUDGET && M * 5 < tiled * 4 && nmat >= 256 && nmat <= 0x7fffffff) {
                permute_matrices_kernel<T><<<(unsigned)nmat, 256, 0, stream>>>((const T*)src, (T*)dst, (int)n0, (int)n1, (int)pitch);
                RK_LAUNCH_CHECK();
                return RK_SUCCESS;
            }
        }
    }
    if constexpr (E <= 8) {
        constexpr int V = 16 / E;
        if (is_aligned(src, 16) && is_aligned(dst, 16) && g.ext[0] % V == 0 && g.ext[g.p] % V == 0) {
            constexpr int TE = E <= 2 ? 128 : 64;
            const int64_t tiles0 = (g.ext[0] + TE - 1) / TE, tilesp = (g.ext[g.p] + TE - 1) / TE;
            int64_t batch = 1;
            for (int d = 1; d < g.nd; ++d)
                if (d != g.p) batch *= g.ext[d];
            // bands of tile rows for the 8 XCDs (see the kernel) unless the pitch asks for the diagonal order or too many workgroups would be empty
            const int64_t rows8 = (tilesp + PERM_XCDS - 1) / PERM_XCDS * PERM_XCDS;
            const int64_t cols8 = (tiles0 + PERM_XCDS - 1) / PERM_XCDS * PERM_XCDS;
            const bool off4k = (g.dstride[0] * (int64_t)E) % 4096 != 0;
            const int by_xcd = off4k && rows8 * 7 <= tilesp * 8 ? 1 : (off4k && tilesp < PERM_XCDS && tiles0 >= 64 ? 2 : 0);
            const int64_t nrows = by_xcd == 1 ? rows8 : tilesp, ncols = by_xcd == 2 ? cols8 : tiles0;
            if (ncols > 0x7fffffff / nrows || ncols * nrows > 0x7fffffff / batch) return RK_ERR_TOO_LARGE;
            permute_tiles_vec_kernel<T, TE, false><<<(unsigned)(ncols * nrows * batch), 256, 0, stream>>>((const T*)src, (T*)dst, g, tiles0, tilesp, by_xcd);
            RK_LAUNCH_CHECK();
            return RK_SUCCESS;
        }
        if constexpr (E >= 4) {
            if (g.ext[0] >= V && g.ext[g.p] >= V) {      // odd extents or addresses: the same tiles, element-aligned vectors
                constexpr int TE = 64;
                const int64_t tiles0 = (g.ext[0] + TE - 1) / TE, tilesp = (g.ext[g.p] + TE - 1) / TE;
                int64_t batch = 1;
                for (int d = 1; d < g.nd; ++d)
                    if (d != g.p) batch *= g.ext[d];
                const int64_t rows8 = (tilesp + PERM_XCDS - 1) / PERM_XCDS * PERM_XCDS;
                const int64_t cols8 = (tiles0 + PERM_XCDS - 1) / PERM_XCDS * PERM_XCDS;
                const bool off4k = (g.dstride[0] * (int64_t)E) % 4096 != 0;
                const int by_xcd = off4k && rows8 * 7 <= tilesp * 8 ? 1 : (off4k && tilesp < PERM_XCDS && tiles0 >= 64 ? 2 : 0);
                const int64_t nrows = by_xcd == 1 ? rows8 : tilesp, ncols = by_xcd == 2 ? cols8 : tiles0;
                if (ncols > 0x7fffffff / nrows || ncols * nrows > 0x7fffffff / batch) return RK_ERR_TOO_LARGE;
                permute_tiles_vec_kernel<T, TE, true><<<(unsigned)(ncols * nrows * batch), 256, 0, stream>>>((const T*)src, (T*)dst, g, tiles0, tilesp, by_xcd);
                RK_LAUNCH_CHECK();
                return RK_SUCCESS;
            }
        }
    }
    constexpr int PT = E == 16 ? 32 : 64;
    const int64_t tiles0 = (g.ext[0] + PT - 1) / PT, tilesp = (g.ext[g.p] + PT - 1) / PT;
    int64_t batch = 1;
    for (int d = 1; d < g.nd; ++d)
        if (d != g.p) batch *= g.ext[d];
    if (tiles0 > 0x7fffffff / tilesp || tiles0 * tilesp > 0x7fffffff / batch) return RK_ERR_TOO_LARGE;
    permute_tiles_kernel<T, PT><<<(unsigned)(tiles0 * tilesp * batch), 256, 0, stream>>>((const T*)src, (T*)dst, g, tiles0, tilesp);
    RK_LAUNCH_CHECK();
    return RK_SUCCESS;
}

}  // namespace rk

using namespace rk;

extern "C" int32_t rk_permutedims(const void* src, void* dst, size_t elsize, int ndim, const int64_t* shape, const int32_t* perm,
                                  void* stream) {
    if (ndim < 0 || ndim > RK_MAX_DIMS || (ndim > 0 && (shape == nullptr || perm == nullptr))) return RK_ERR_INVALID_ARGUMENT;
    if (elsize != 1 && elsize != 2 && elsize != 4 && elsize != 8 && elsize != 16) return RK_ERR_UNSUPPORTED;
    int64_t total = 1;
    uint32_t seen = 0;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] < 0) return RK_ERR_INVALID_ARGUMENT;
        if (shape[d] != 0 && total > INT64_MAX / shape[d]) return RK_ERR_INVALID_ARGUMENT;
        total *= shape[d];
        if (perm[d] < 1 || perm[d] > ndim || (seen >> (perm[d] - 1) & 1u)) return RK_ERR_INVALID_ARGUMENT;   // not a permutation
        seen |= 1u << (perm[d] - 1);
    }
    if (total == 0) return RK_SUCCESS;
    if (src == nullptr || dst == nullptr || src == dst) return RK_ERR_INVALID_ARGUMENT;
    const size_t align = elsize < 16 ? elsize : 8;
    if (!is_aligned(src, align) || !is_aligned(dst, align)) return RK_ERR_INVALID_ARGUMENT;
    // dst dims in order, without extents of 1; neighbours that are neighbours in src too are merged
    int order[RK_MAX_DIMS];          // src dim (0-based) of every kept dst position
    int n = 0;
    for (int k = 0; k < ndim; ++k)
        if (shape[perm[k] - 1] != 1) order[n++] = perm[k] - 1;
    // merged src dims: runs of consecutive kept src dims that appear consecutively in `order`
    int group_of[RK_MAX_DIMS];       // src dim -> merged dim
    bool head[RK_MAX_DIMS] = {};     // src dim starts a merged dim
    for (int k = 0; k < n; ++k) {
        bool joins = false;          // order[k] continues the run of order[k-1]?
        if (k > 0 && order[k] > order[k - 1]) {
            joins = true;
            for (int d = order[k - 1] + 1; d < order[k]; ++d)
                if (shape[d] != 1) joins = false;
        }
        head[order[k]] = !joins;
    }
    PermGeom g{};
    g.total = total;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] == 1) continue;
        if (head[d]) { g.ext[g.nd] = shape[d]; group_of[d] = g.nd++; }
        else { g.ext[g.nd - 1] *= shape[d]; group_of[d] = g.nd - 1; }
    }
    if (g.nd == 0) { g.ext[0] = 1; g.nd = 1; g.dstride[0] = 1; g.p = 0; }
    else {
        int64_t stride = 1;
        bool first = true;
        for (int k = 0; k < n; ++k) {
            if (!head[order[k]]) continue;
            const int m = group_of[order[k]];
            g.dstride[m] = stride;
            stride *= g.ext[m];
            if (first) { g.p = m; first = false; }
        }
    }
    hipStream_t st = (hipStream_t)stream;
    switch (elsize) {
        case 1: return permute_elsize<1>(src, dst, g, st);
        case 2: return permute_elsize<2>(src, dst, g, st);
        case 4: return permute_elsize<4>(src, dst, g, st);
        case 8: return permute_elsize<8>(src, dst, g, st);
        default: return permute_elsize<16>(src, dst, g, st);
    }
}
