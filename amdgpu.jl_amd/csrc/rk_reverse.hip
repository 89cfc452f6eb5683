// reverse / reverse! along any set of dimensions (src/kernels/reverse.jl:59-122), for any element size.
//
// The host merges neighbouring dimensions that are flipped alike (flipping two adjacent dims of a dense array
// is flipping the merged one) and drops extents of 1, then the array is moved in units: 16-byte units when the
// rows are whole units and everything is 16-byte aligned (a flipped first dimension then also reverses the
// elements inside the unit), single elements otherwise.  One unit per lane: loads are coalesced, stores are
// coalesced in the flipped direction.  8 bytes per byte-pair moved, no workspace.
#include "rk_common.hpp"

namespace rk {

struct RevGeom {
    int64_t ext[RK_MAX_DIMS];   // extents of the merged dims, dim 0 in units
    int64_t total;              // units
    uint32_t flip;              // bit d: merged dim d is flipped
    int nd;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Reverses the E-byte elements inside a 16-byte unit.
template <int E>
__device__ __forceinline__ u32x4 flip_unit(u32x4 v) {
    if constexpr (E == 16) return v;
    else if constexpr (E == 8) return u32x4{v[2], v[3], v[0], v[1]};
    else if constexpr (E == 4) return u32x4{v[3], v[2], v[1], v[0]};
    else if constexpr (E == 2) {
        return u32x4{(v[3] >> 16) | (v[3] << 16), (v[2] >> 16) | (v[2] << 16), (v[1] >> 16) | (v[1] << 16), (v[0] >> 16) | (v[0] << 16)};
    } else {
        return u32x4{__builtin_bswap32(v[3]), __builtin_bswap32(v[2]), __builtin_bswap32(v[1]), __builtin_bswap32(v[0])};
    }
}

template <int E> struct ElemOf;
template <> struct ElemOf<1> { typedef uint8_t type; };
template <> struct ElemOf<2> { typedef uint16_t type; };
template <> struct ElemOf<4> { typedef uint32_t type; };
template <> struct ElemOf<8> { typedef uint64_t type; };
template <> struct ElemOf<16> { struct type { uint64_t lo, hi; }; };

// Index of the unit that unit `i` moves to.
template <typename I>
__device__ __forceinline__ int64_t flipped_index(I i, const RevGeom& g) {
    I rem = i, out = 0, stride = 1;
    for (int d = 0; d < g.nd; ++d) {
        const I e = (I)g.ext[d];
        I c;
        if (d == g.nd - 1) c = rem;
        else { const I q = rem / e; c = rem - q * e; rem = q; }
        if (g.flip >> d & 1u) c = e - 1 - c;
        out += c * stride;
        stride *= e;
    }
    return (int64_t)out;
}

// UNIT: the moved unit (u32x4 or the element type); FLIP_IN_UNIT: element size when units are 16 bytes and dim 0
// is flipped (0 = leave the unit as it is); INPLACE: y == x, pairs are swapped by the lane with the lower index.
// 16-byte units stream through with non-temporal accesses (nothing is read twice); elements take plain ones.
template <typename UNIT> __device__ __forceinline__ UNIT rev_load(const UNIT* p) { return *p; }
template <typename UNIT> __device__ __forceinline__ void rev_store(UNIT* p, UNIT v) { *p = v; }
template <> __device__ __forceinline__ u32x4 rev_load<u32x4>(const u32x4* p) { return load_nt(p); }
template <> __device__ __forceinline__ void rev_store<u32x4>(u32x4* p, u32x4 v) { store_nt(p, v); }

template <typename UNIT, int FLIP_IN_UNIT, bool INPLACE, typename I>
__global__ __launch_bounds__(256) void reverse_kernel(const UNIT* __restrict__ x, UNIT* __restrict__ y, RevGeom g) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= g.total) return;
    const int64_t o = flipped_index<I>((I)i, g);
    if constexpr (!INPLACE) {
        UNIT v = rev_load(x + i);
        if constexpr (FLIP_IN_UNIT != 0) v = flip_unit<FLIP_IN_UNIT>(v);
        rev_store(y + o, v);
    } else {
        UNIT* p = y;        // x and y are the same array: go through one pointer
        if (i > o) return;
        UNIT a = rev_load(p + i);
        if constexpr (FLIP_IN_UNIT != 0) a = flip_unit<FLIP_IN_UNIT>(a);
        if (i == o) { rev_store(p + i, a); return; }
        UNIT b = rev_load(p + o);
        if constexpr (FLIP_IN_UNIT != 0) b = flip_unit<FLIP_IN_UNIT>(b);
        rev_store(p + o, a);
        rev_store(p + i, b);
    }
}

template <typename UNIT, int FLIP_IN_UNIT>
static int32_t launch_reverse(const void* x, void* y, const RevGeom& g, hipStream_t stream) {
    const int64_t blocks = (g.total + 255) / 256;
    if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
    const bool small = g.total <= 0xffffffffll;
    const bool inplace = (x == y);
#define RK_REV(INP, IT) reverse_kernel<UNIT, FLIP_IN_UNIT, INP, IT><<<(unsigned)blocks, 256, 0, stream>>>((const UNIT*)x, (UNIT*)y, g)
    if (inplace) { if (small) RK_REV(true, uint32_t); else RK_REV(true, uint64_t); }
    else         { if (small) RK_REV(false, uint32_t); else RK_REV(false, uint64_t); }
#undef RK_REV
    RK_LAUNCH_CHECK();
    return RK_SUCCESS;
}

// ---- rows that are no whole number of 16-byte units (reverse(A; dims=1) of a 1001 x N Float32 array) ----------------
// One element per lane moves 4 bytes a lane, 3 TB/s.  Global memory takes 16-byte accesses at any element-aligned
// address (only LDS wants them aligned to their size), so a lane moves a group of 16 / E consecutive elements of a row
// with one load and one store, neither 16-byte aligned in general; a flipped first dim reverses the elements inside
// the group.  The last group of a row, when it is short, goes element by element.  Out of place only.
template <int E> struct GroupOf;
template <> struct GroupOf<4> { typedef uint32_t elem; typedef uint32_t type __attribute__((ext_vector_type(4), aligned(4))); };
template <> struct GroupOf<8> { typedef uint64_t elem; typedef uint64_t type __attribute__((ext_vector_type(2), aligned(8))); };

template <int E, typename I>
__global__ __launch_bounds__(256) void reverse_groups_kernel(const typename GroupOf<E>::elem* __restrict__ x,
                                                             typename GroupOf<E>::elem* __restrict__ y, RevGeom g, int64_t groups_per_row,
                                                             int64_t ngroups) {
    typedef typename GroupOf<E>::type G;
    constexpr int N = 16 / E;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= ngroups) return;
    const I ext0 = (I)g.ext[0];
    const I row = (I)i / (I)groups_per_row, q = (I)i - row * (I)groups_per_row;
    const I c0 = q * N;
    const int n = ext0 - c0 < (I)N ? (int)(ext0 - c0) : N;
    // the row the row moves to: dims 1 .. nd-1 flipped like flipped_index does
    I rem = row, orow = 0, stride = 1;
    for (int d = 1; d < g.nd; ++d) {
        const I e = (I)g.ext[d];
        I c;
        if (d == g.nd - 1) c = rem;
        else { const I qd = rem / e; c = rem - qd * e; rem = qd; }
        if (g.flip >> d & 1u) c = e - 1 - c;
        orow += c * stride;
        stride *= e;
    }
    const bool flip0 = g.flip & 1u;
    const int64_t src = (int64_t)row * (int64_t)ext0 + (int64_t)c0;
    const int64_t dst = (int64_t)orow * (int64_t)ext0 + (int64_t)(flip0 ? ext0 - c0 - (I)n : c0);
    if (n == N) {
        G v = __builtin_nontemporal_load((const G*)(x + src));
        if (flip0) {
            if constexpr (N == 4) v = G{v[3], v[2], v[1], v[0]};
            else v = G{v[1], v[0]};
        }
        __builtin_nontemporal_store(v, (G*)(y + dst));
    } else {
        for (int j = 0; j < n; ++j) y[dst + (flip0 ? n - 1 - j : j)] = x[src + j];
    }
}

template <int E>
static int32_t launch_reverse_groups(const void* x, void* y, const RevGeom& g, hipStream_t stream) {
    constexpr int N = 16 / E;
    const int64_t groups_per_row = (g.ext[0] + N - 1) / N, rows = g.total / g.ext[0];
    if (rows != 0 && groups_per_row > INT64_MAX / rows) return RK_ERR_TOO_LARGE;
    const int64_t ngroups = groups_per_row * rows, blocks = (ngroups + 255) / 256;
    if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
    typedef typename GroupOf<E>::elem elem;
    if (g.total <= 0x7fffffffll)
        reverse_groups_kernel<E, uint32_t><<<(unsigned)blocks, 256, 0, stream>>>((const elem*)x, (elem*)y, g, groups_per_row, ngroups);
    else
        reverse_groups_kernel<E, int64_t><<<(unsigned)blocks, 256, 0, stream>>>((const elem*)x, (elem*)y, g, groups_per_row, ngroups);
    RK_LAUNCH_CHECK();
    return RK_SUCCESS;
}

template <int E>
static int32_t reverse_elsize(const void* x, void* y, RevGeom g, bool vector, hipStream_t stream) {
    if constexpr (E == 4 || E == 8) {
        if (!vector && x != y && g.ext[0] >= 16 / E) return launch_reverse_groups<E>(x, y, g, stream);
    }
    if (vector) {
        g.ext[0] = g.ext[0] * E / 16;
        g.total = g.total * E / 16;
        if (g.flip & 1u) return launch_reverse<u32x4, E>(x, y, g, stream);
        return launch_reverse<u32x4, 0>(x, y, g, stream);
    }
    return launch_reverse<typename ElemOf<E>::type, 0>(x, y, g, stream);
}

}  // namespace rk

using namespace rk;

extern "C" int32_t rk_reverse(const void* x, void* y, size_t elsize, int ndim, const int64_t* shape, uint32_t rev_mask, void* stream) {
    if (ndim < 0 || ndim > RK_MAX_DIMS || (ndim > 0 && shape == nullptr)) return RK_ERR_INVALID_ARGUMENT;
    if (elsize != 1 && elsize != 2 && elsize != 4 && elsize != 8 && elsize != 16) return RK_ERR_UNSUPPORTED;
    int64_t total = 1;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] < 0) return RK_ERR_INVALID_ARGUMENT;
        if (shape[d] != 0 && total > INT64_MAX / shape[d]) return RK_ERR_INVALID_ARGUMENT;
        total *= shape[d];
    }
    if (total == 0) return RK_SUCCESS;
    if (x == nullptr || y == nullptr) return RK_ERR_INVALID_ARGUMENT;
    // merge: drop extents of 1, fuse neighbours with the same flip flag (reverse.jl:67: dims of extent 1 never flip)
    RevGeom g{};
    g.total = total;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] == 1) continue;
        const uint32_t f = (rev_mask >> d) & 1u;
        if (g.nd > 0 && ((g.flip >> (g.nd - 1)) & 1u) == f) g.ext[g.nd - 1] *= shape[d];
        else {
            g.ext[g.nd] = shape[d];
            g.flip |= f << g.nd;
            ++g.nd;
        }
    }
    if (g.nd == 0) { g.ext[0] = 1; g.nd = 1; }                   // a single element
    if (x == y && g.flip == 0u) return RK_SUCCESS;               // reverse! of nothing
    const size_t align = elsize < 16 ? elsize : 8;
    if (!is_aligned(x, align) || !is_aligned(y, align)) return RK_ERR_INVALID_ARGUMENT;
    const bool vector = is_aligned(x, 16) && is_aligned(y, 16) && (g.ext[0] * (int64_t)elsize) % 16 == 0;
    hipStream_t st = (hipStream_t)stream;
    switch (elsize) {
        case 1: return reverse_elsize<1>(x, y, g, vector, st);
        case 2: return reverse_elsize<2>(x, y, g, vector, st);
        case 4: return reverse_elsize<4>(x, y, g, vector, st);
        case 8: return reverse_elsize<8>(x, y, g, vector, st);
        default: return reverse_elsize<16>(x, y, g, vector, st);
    }
}
