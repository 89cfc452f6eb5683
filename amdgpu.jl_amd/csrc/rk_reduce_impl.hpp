// Reduction kernels: mapreduce over all / some dimensions of a column-major array, and the
// (value, index) reductions of findmax / findmin.  Replaces partial_mapreduce_device and
// reduce_group of the reference (src/kernels/mapreduce.jl:43-82, :8-34) and the host driver
// mapreducedim! (:86-173): one launch, no recursion, no temporary allocation.
//
// A reduction over one run of adjacent dimensions sees the array as (inner, mid, outer) with
// `mid` reduced.  Output q = i + inner * o is the reduction of the "line"
//     A[i + inner * (m + mid * o)],  m = 0 .. mid-1          (element stride `inner`).
// Four kernels cover the shapes:
//   reduce_split_kernel    few long lines (incl. the full reduction): `splits` workgroups per
//                          line, 128-bit loads when the line is contiguous, partials + a
//                          completion ticket, the last workgroup of a line combines them in a
//                          fixed order (deterministic, single launch)
//   reduce_wave_kernel     many medium lines: one wave per line, no LDS, no barrier
//   reduce_thread_kernel   very many tiny lines: one lane per line
//   reduce_short_lines_kernel  many short lines (contiguous, or inner < 64): whole inner x mid slabs through LDS
//   reduce_narrow_kernel   1 < inner < 64 with long lines: contiguous runs of whole rows
//   reduce_strided_kernel  inner >= 64: lanes run along the contiguous `inner` axis (128-bit
//                          loads), waves and workgroups split `mid`
// plus reduce_generic_kernel for masks that are not one run (e.g. dims=(1,3)).
#pragma once

#include "rk_common.hpp"
#include "rk_interp.hpp"

namespace rk {

struct LineGeom {
    int64_t inner;   // lines per outer slab == element stride along a line
    int64_t mid;     // line length
    int64_t nlines;  // inner * outer
};

__device__ __forceinline__ int64_t line_base(const LineGeom& g, int64_t q) {
    if (g.inner == 1) return q * g.mid;
    const int64_t o = q / g.inner, i = q - o * g.inner;
    return i + o * g.inner * g.mid;
}

// ---- element transforms ---------------------------------------------------------------------
// Called as xf(value, position along the line).  f is applied in the input type, then converted
// (Julia: add_sum(widen(f(x)))).
template <typename In, typename Acc, typename Map> struct MapXform {
    typedef int64_t Pos;
    __device__ __forceinline__ Acc operator()(In x, int64_t) const { return (Acc)Map()(x); }
};
template <typename T, typename P> using ArgAcc = KeyIdx<typename OrderKey<T>::Key, P, OrderKey<T>::LOWEST_FREE>;
template <typename T, typename P, bool WANT_MAX> struct ArgXform {
    typedef P Pos;
    typedef ArgAcc<T, P> A;
    __device__ __forceinline__ A operator()(T x, P pos) const { A p; p.k = OrderKey<T>::make(x, WANT_MAX); p.i = pos; return p; }
};

// f given as a postfix program over the element (operand token 0) and up to RK_MAP_MAX_CONSTS constants (tokens
// 1 ..): mapreduce(x -> x + 1, +, A), count(isodd, A).  Floating-point elements compute in their own type, integers
// in Int64 (the program wraps to 32 bits itself where Julia's value would).  The interpreter costs one scalar
// branch per token, so the kernels hand it the values of one or two vector loads at a time (`batch`).
struct PackedTokens {                        // 16 tokens of 8 bits in two scalar registers: no memory behind tokens[i]
    uint64_t lo, hi;
    __device__ __forceinline__ int operator[](int i) const { return (int)(((i < 8 ? lo : hi) >> ((i & 7) * 8)) & 0xffu); }
};
template <typename In, typename Acc> struct ProgXform {
    typedef int64_t Pos;
    typedef typename std::conditional<std::is_floating_point<In>::value, In, int64_t>::type CT;
    static constexpr int CHUNK = 32 / sizeof(CT);        // components per interpreter run: 8 Float32, 4 Float64 / Int64
    PackedTokens tokens;
    int32_t n_tokens;
    CT c[RK_MAP_MAX_CONSTS];
    template <int N> struct Fetch {
        static constexpr int NOPS = 1 + RK_MAP_MAX_CONSTS;
        const In* x;
        const CT (&c)[RK_MAP_MAX_CONSTS];
        template <int K> __device__ __forceinline__ void get(CT (&v)[N]) const {
#pragma unroll
            for (int j = 0; j < N; ++j) {
                if constexpr (K == 0) v[j] = (CT)x[j];
                else v[j] = c[K - 1];
            }
        }
    };
    template <int N> __device__ __forceinline__ void batch(const In* x, Acc* y) const {
        CT out[N];
        interp_run<CT, N, 0, false>(tokens, n_tokens, Fetch<N>{x, c}, out, (CT*)nullptr);
#pragma unroll
        for (int j = 0; j < N; ++j) y[j] = (Acc)out[j];
    }
    __device__ __forceinline__ Acc operator()(In x, int64_t) const {
        Acc y;
        batch<1>(&x, &y);
        return y;
    }
};
// f = one arithmetic operator between the element and a constant -- x + c, c + x, x - c, c - x, x * c, c * x; the
// reference's own benchmark closure is x -> x + 1 (perf/array.jl:107-122) -- needs no interpreter: it is x * m + a
// with (m, a) = (1, c), (1, -c), (-1, c), (c, -0.0).  Each of these is the operator's own value bit for bit, fused or
// not: a product with +-1 is exact, x - c is x + (-c) in IEEE arithmetic, and adding -0.0 changes nothing, not even
// the sign of a zero.  Integers wrap in 64 bits like the interpreter's.
template <typename In, typename Acc> struct AffineXform {
    typedef int64_t Pos;
    typedef typename ProgXform<In, Acc>::CT CT;
    CT m, a;
    __device__ __forceinline__ Acc operator()(In x, int64_t) const {
        if constexpr (std::is_integral<CT>::value) return (Acc)wrap_add(wrap_mul((CT)x, m), a);
        else return (Acc)((CT)x * m + a);
    }
};
template <typename Xf> struct XfIsArg : std::false_type {};
template <typename T, typename P, bool WANT_MAX> struct XfIsArg<ArgXform<T, P, WANT_MAX>> : std::true_type {};
template <typename Xf> struct XfIsBatch : std::false_type {};
template <typename In, typename Acc> struct XfIsBatch<ProgXform<In, Acc>> : std::true_type {};

// m[i] = xf(x[i]) for TOTAL loaded values, CHUNK at a time
template <int TOTAL, typename In, typename Acc, typename Xf>
__device__ __forceinline__ void map_batch(const In (&x)[TOTAL], Acc (&m)[TOTAL], const Xf& xf) {
    constexpr int C = TOTAL < Xf::CHUNK ? TOTAL : Xf::CHUNK;
    static_assert(TOTAL % C == 0, "loaded values split into whole chunks");
#pragma unroll
    for (int c0 = 0; c0 < TOTAL; c0 += C) xf.template batch<C>(&x[c0], &m[c0]);
}

// ---- result sinks ---------------------------------------------------------------------------
// Called as sink(output index q, reduced value).
// Out differs from Acc for Float16 arrays (accumulated in Float32, rounded once at the end).
template <typename Acc, typename Op, typename Out = Acc> struct ReduceSink {
    Out* R;
    Acc  init;
    int  has_init;
    __device__ __forceinline__ void operator()(int64_t q, Acc t) const { R[q] = (Out)(has_init ? Op()(init, t) : t); }
};
// The value written is the winning ELEMENT, read back from A at the winner's position: decoding the key would turn
// every NaN into the canonical one, and Julia returns the element itself (sign and payload of a NaN included).
template <typename T, typename P> struct ArgSink {
    const T* A;
    T*       vals;
    int64_t* cart;
    int      ndim;
    int64_t  shape[RK_MAX_DIMS];
    bool     want_max;
    bool     absolute;   // positions are already linear offsets into A (the generic kernel)
    int8_t   slot[RK_MAX_DIMS];   // component of the CartesianIndex that dim d of `shape` fills (d itself; a wrapper's logical dim)
    LineGeom g;
    __device__ __forceinline__ void operator()(int64_t q, ArgAcc<T, P> t) const {
        const int64_t lin = absolute ? (int64_t)t.i : line_base(g, q) + (int64_t)t.i * g.inner;
        if (vals) vals[q] = t.i < 0 ? OrderKey<T>::value(t.k, want_max) : A[lin];
        if (cart) {
            int64_t rem = lin;
            for (int d = 0; d < ndim; ++d) {
                const int64_t c = rem % shape[d];
                rem /= shape[d];
                cart[q * ndim + slot[d]] = c + 1;
            }
        }
    }
};

// ---- accumulate one slice of one line with GROUP cooperating threads --------------------------
// slice s of `splits`; `t` = thread index inside the group.  Contiguous lines are read as
// 16-byte vectors after peeling the unaligned head.
template <typename In, typename Acc, typename Xf, typename Op, bool VECTOR, int GROUP, int UNROLL>
__device__ __forceinline__ Acc accumulate_line(const In* __restrict__ A, int64_t base, int64_t n, int64_t stride,
                                               int s, int splits, int t, Xf xf, Op op) {
    typedef typename Xf::Pos Pos;
    if constexpr (VECTOR) {
        constexpr int VEC = 16 / sizeof(In);
        typedef typename VecOf<In, VEC>::type V;
        Acc acc[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] = Op::template identity<Acc>();
        const In* p = A + base;
        int64_t head = (int64_t)(((16 - ((uintptr_t)p & 15)) & 15) / sizeof(In));
        if (head > n) head = n;
        const int64_t nvec = (n - head) / VEC;
        const V* pv = (const V*)(p + head);
        const int64_t tail = head + nvec * VEC;
        Acc edge = Op::template identity<Acc>();   // kept apart: the vector body below must see increasing indices
        if (s == 0) {   // fewer than VEC (<= 16 <= GROUP) scalars on either side
            if (t < head) edge = op(edge, xf(p[t], (Pos)t));
            if (tail + t < n) edge = op(edge, xf(p[tail + t], (Pos)(tail + t)));
        }
        constexpr int64_t CHUNK = (int64_t)GROUP * UNROLL;
        const int64_t nchunks = nvec / CHUNK;
        for (int64_t c = s; c < nchunks; c += splits) {
            V v[UNROLL];
            const int64_t i0 = c * CHUNK + t;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) v[u] = load_nt(pv + i0 + (int64_t)u * GROUP);
            if constexpr (XfIsBatch<Xf>::value) {
                In x[UNROLL * VEC];
                Acc m[UNROLL * VEC];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u)
#pragma unroll
                    for (int j = 0; j < VEC; ++j) x[u * VEC + j] = v[u][j];
                map_batch<UNROLL * VEC>(x, m, xf);
#pragma unroll
                for (int u = 0; u < UNROLL; ++u)
#pragma unroll
                    for (int j = 0; j < VEC; ++j) acc[j] = acc_step(op, acc[j], m[u * VEC + j]);
            } else {
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const Pos e0 = (Pos)(head + (i0 + (int64_t)u * GROUP) * VEC);
#pragma unroll
                    for (int j = 0; j < VEC; ++j) acc[j] = acc_step(op, acc[j], xf(v[u][j], (Pos)(e0 + j)));
                }
            }
        }
        for (int64_t i = nchunks * CHUNK + (int64_t)s * GROUP + t; i < nvec; i += (int64_t)splits * GROUP) {
            const V v = load_nt(pv + i);
            const Pos e0 = (Pos)(head + i * VEC);
            if constexpr (XfIsBatch<Xf>::value) {
                In x[VEC];
                Acc m[VEC];
#pragma unroll
                for (int j = 0; j < VEC; ++j) x[j] = v[j];
                map_batch<VEC>(x, m, xf);
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[j] = acc_step(op, acc[j], m[j]);
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[j] = acc_step(op, acc[j], xf(v[j], (Pos)(e0 + j)));
            }
        }
        Acc a = edge;
#pragma unroll
        for (int j = 0; j < VEC; ++j) a = op(a, acc[j]);
        return a;
    } else {
        Acc acc[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) acc[u] = Op::template identity<Acc>();
        const int64_t step = (int64_t)splits * GROUP;
        int64_t k = (int64_t)s * GROUP + t;
        for (; k + (UNROLL - 1) * step < n; k += UNROLL * step) {
            In v[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) v[u] = A[base + (k + u * step) * stride];
            if constexpr (XfIsBatch<Xf>::value) {
                Acc m[UNROLL];
                map_batch<UNROLL>(v, m, xf);
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) acc[u] = acc_step(op, acc[u], m[u]);
            } else {
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) acc[u] = acc_step(op, acc[u], xf(v[u], (Pos)(k + u * step)));
            }
        }
        for (; k < n; k += step) acc[0] = acc_step(op, acc[0], xf(A[base + k * stride], (Pos)k));
        Acc a = acc[0];
#pragma unroll
        for (int u = 1; u < UNROLL; ++u) a = op(a, acc[u]);
        return a;
    }
}

// ---- few long lines: grid (splits, nlines) ---------------------------------------------------
template <typename In, typename Acc, typename Xf, typename Op, typename Sink, bool VECTOR, int BLOCK, int UNROLL>
__global__ __launch_bounds__(BLOCK) void reduce_split_kernel(const In* __restrict__ A, LineGeom g, Xf xf, Op op, Sink sink,
                                                             Acc* partials, uint32_t* tickets) {
    constexpr int NW = BLOCK / WAVE;
    __shared__ Acc lds[NW];
    __shared__ int is_last;
    const int s = blockIdx.x, splits = gridDim.x, t = threadIdx.x;
    const int64_t line = blockIdx.y;
    const int64_t base = line_base(g, line);
    Acc a = accumulate_line<In, Acc, Xf, Op, VECTOR, BLOCK, UNROLL>(A, base, g.mid, g.inner, s, splits, t, xf, op);
    a = block_reduce<NW>(a, op, lds);
    if (splits == 1) {
        if (t == 0) sink(line, a);
        return;
    }
    // Two levels of completion tickets.  Device-wide atomics on ONE address complete at roughly 14 ns each
    // on MI355X, so thousands of workgroups must not share a ticket: groups of TICKET_GROUP workgroups
    // share one (each on its own 128-byte line), the last arrival of a group folds the group's partials
    // in lane order and takes a ticket of the line, the last group folds the group results.  All orders
    // are fixed, so the result does not depend on arrival order.
    const int ngroups = (splits + TICKET_GROUP - 1) / TICKET_GROUP;
    const int grp = s / TICKET_GROUP;
    const int gsize = (grp == ngroups - 1) ? splits - grp * TICKET_GROUP : TICKET_GROUP;
    Acc* gpartials = partials + (int64_t)gridDim.y * splits;
    uint32_t* gticket = tickets + (line * (ngroups + 1) + grp) * TICKET_STRIDE;
    uint32_t* lticket = tickets + (line * (ngroups + 1) + ngroups) * TICKET_STRIDE;
    if (t == 0) {
        store_agent(&partials[line * splits + s], a);
        publish_barrier();      // the partial is at the coherent level before the ticket moves
        const uint32_t old = __hip_atomic_fetch_add(gticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        is_last = (old == (uint32_t)gsize - 1u);
    }
    __syncthreads();
    if (!is_last) return;
    __syncthreads();            // everybody has read is_last before it is written again
    if (t < WAVE) {
        static_assert(TICKET_GROUP <= WAVE, "a group is folded by one wave");
        Acc r = t < gsize ? load_agent(&partials[line * splits + grp * TICKET_GROUP + t]) : Op::template identity<Acc>();
        r = wave_reduce(r, op);
        if (t == 0) {
            *gticket = 0;       // leave the workspace clean for the next call
            store_agent(&gpartials[line * ngroups + grp], r);
            publish_barrier();
            const uint32_t old = __hip_atomic_fetch_add(lticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            is_last = (old == (uint32_t)ngroups - 1u);
        }
    }
    __syncthreads();
    if (!is_last) return;
    Acc r = Op::template identity<Acc>();
    for (int i = t; i < ngroups; i += BLOCK) r = op(r, load_agent(&gpartials[line * ngroups + i]));
    r = block_reduce<NW>(r, op, lds);
    if (t == 0) {
        sink(line, r);
        *lticket = 0;
    }
}

// ---- many medium lines: one wave per line ------------------------------------------------------
template <typename In, typename Acc, typename Xf, typename Op, typename Sink, bool VECTOR, int BLOCK, int UNROLL>
__global__ __launch_bounds__(BLOCK) void reduce_wave_kernel(const In* __restrict__ A, LineGeom g, Xf xf, Op op, Sink sink) {
    const int64_t line = (int64_t)blockIdx.x * (BLOCK / WAVE) + threadIdx.x / WAVE;
    if (line >= g.nlines) return;
    const int64_t base = line_base(g, line);
    Acc a = accumulate_line<In, Acc, Xf, Op, VECTOR, WAVE, UNROLL>(A, base, g.mid, g.inner, 0, 1, lane_id(), xf, op);
    a = wave_reduce(a, op);
    if (lane_id() == 0) sink(line, a);
}

// ---- very many tiny lines: one lane per line -----------------------------------------------------
template <typename In, typename Acc, typename Xf, typename Op, typename Sink, int BLOCK>
__global__ __launch_bounds__(BLOCK) void reduce_thread_kernel(const In* __restrict__ A, LineGeom g, Xf xf, Op op, Sink sink) {
    const int64_t line = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (line >= g.nlines) return;
    const int64_t base = line_base(g, line);
    Acc a = Op::template identity<Acc>();
    for (int64_t k = 0; k < g.mid; ++k) a = acc_step(op, a, xf(A[base + k * g.inner], (typename Xf::Pos)k));
    sink(line, a);
}

// ---- a short reduced dim behind a long contiguous one: a lane per group of columns ------------------------------
// (sum(A; dims=2) of a 200 x 3 x 50000 or a 50000 x 3 x 200 array: the strided kernel gave every workgroup three rows
// of a strip -- 39200 workgroups for 2.4 KB each, 2.4 TB/s; a lane per line reads 4 bytes at a time.)  A lane owns
// VEC = 16 / sizeof(In) adjacent columns of one outer index and walks the <= 16 rows with 16-byte loads at
// element-aligned addresses, four in flight; the last group of a row starts VEC columns before the row's end and
// drops the columns it shares with the group before.  4- and 8-byte elements, inner >= VEC.
template <typename In, typename Acc, typename Xf, typename Op, typename Sink>
__global__ __launch_bounds__(256) void reduce_cols_kernel(const In* __restrict__ A, LineGeom g, Xf xf, Op op, Sink sink,
                                                          int64_t groups_per_row, int64_t ngroups) {
    constexpr int VEC = 16 / sizeof(In);
    typedef typename VecOf<In, VEC>::type V;
    typedef typename Xf::Pos Pos;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= ngroups) return;
    const int64_t o = i / groups_per_row, q = i - o * groups_per_row;
    const int64_t nominal = q * VEC;
    const int64_t col0 = nominal + VEC > g.inner ? g.inner - VEC : nominal;
    const int dup = (int)(nominal - col0);
    const In* p = A + o * g.inner * g.mid + col0;
    Acc acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = Op::template identity<Acc>();
    int64_t m = 0;
    for (; m + 4 <= g.mid; m += 4) {
        V v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = load_nt_elems<In, VEC>(p + (m + u) * g.inner);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] = acc_step(op, acc[j], xf(v[u][j], (Pos)(m + u)));
    }
    for (; m < g.mid; ++m) {
        const V v = load_nt_elems<In, VEC>(p + m * g.inner);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] = acc_step(op, acc[j], xf(v[j], (Pos)m));
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        if (j >= dup) sink(o * g.inner + col0 + j, acc[j]);
}

// ---- many short lines, contiguous or with a narrow inner extent: whole slabs through LDS -----------------------
// (sum(A; dims=1) of a 32 x 1_000_000 array; sum(A; dims=2) of a 4 x 32 x 250_000 array.)  A slab is the inner x mid
// block of one outer index, contiguous in memory.  A wave per line leaves most lanes idle or gives each wave too
// little to keep loads in flight, and a lane per line reads with a stride; here a workgroup copies a run of whole
// slabs -- contiguous memory, 16-byte vectors -- into LDS, and a group of tpl = 1, 2, .. 16 lanes folds each line from
// there (lane `part` takes the elements k = part (mod tpl), then a DPP fold across the group).  f is applied on the
// way out of LDS, so LDS holds 1 .. 8 bytes an element whatever the accumulator is (16 for findmax).
// The lines of slab s are walked from element rot(s) with wrap-around (the operators are commutative, and the index
// rule of findmax / findmin does not depend on the order): rot(s) = s * (tpl - m) mod P, P the largest power of two
// <= min(m, 64), puts lane (s, i, part) at an address = inner * (s * tpl + part) + i (mod inner * P), which spreads the
// lanes of a wave over the banks for every m (with inner = 1 a common start is a 32-way conflict for m = 32; s mod m
// is one for m = 31).
// The host picks slabs_per_block so that a block's first element is 16-byte aligned when the array is (VECTOR).
// A traced f (a postfix program) runs while the tile is loaded, and LDS holds its values: Acc-sized slots then.
template <typename In, typename Acc, typename Xf> struct ShortLinesTile {
    static constexpr bool MAPPED_IN_LDS = XfIsBatch<Xf>::value && sizeof(Acc) >= sizeof(In) && sizeof(Acc) <= 8;
    static constexpr int BYTES = 16384;
    static constexpr int ELEMS = BYTES / (MAPPED_IN_LDS ? sizeof(Acc) : sizeof(In));
};
constexpr int SHORT_LINES_MAX = 512;          // contiguous lines beyond this do as well with a wave each (300 elements: 59 us with a wave a line)

template <typename In, typename Acc, typename Xf, typename Op, typename Sink, bool VECTOR>
__global__ __launch_bounds__(256) void reduce_short_lines_kernel(const In* __restrict__ A, int inner, int m, int64_t nslabs, int slabs_per_block,
                                                                 int tpl_log2, int rot_mask, Xf xf, Op op, Sink sink) {
    typedef typename Xf::Pos Pos;
    typedef ShortLinesTile<In, Acc, Xf> Tile;
    __shared__ __attribute__((aligned(16))) char lds_raw[Tile::BYTES];
    In* lds = (In*)lds_raw;
    const int t = threadIdx.x;
    const int slab = inner * m;
    const int64_t slab0 = (int64_t)blockIdx.x * slabs_per_block;
    const int64_t left = nslabs - slab0;
    const int ns = left < slabs_per_block ? (int)left : slabs_per_block;     // > 0 by the grid size
    const int ne = ns * slab;                                                 // <= TE by the choice of slabs_per_block
    const In* p = A + slab0 * slab;
    constexpr int VEC = VECTOR ? 16 / sizeof(In) : 1;
    typedef typename VecOf<In, VEC>::type V;
    const int nv = ne / VEC;
    // A traced f (a postfix program) costs scalar control flow per call, whatever the number of values: it runs here,
    // on two vectors at a time; the fold then reads f's values.
    constexpr bool MAPPED_IN_LDS = Tile::MAPPED_IN_LDS;
    if constexpr (MAPPED_IN_LDS) {
        Acc* mapped = (Acc*)lds_raw;
        if constexpr (VEC == 1) {
            for (int i = t; i < ne; i += 256) mapped[i] = xf(p[i], (Pos)0);
        } else {
            constexpr int AV = 16 / sizeof(Acc);              // <= VEC
            typedef typename VecOf<Acc, AV>::type VA;
            for (int i = t; i < nv; i += 512) {
                const bool second = i + 256 < nv;
                const V v0 = load_nt((const V*)p + i);
                V v1 = v0;
                if (second) v1 = load_nt((const V*)p + i + 256);
                In x[2 * VEC];
                Acc y[2 * VEC];
#pragma unroll
                for (int j = 0; j < VEC; ++j) { x[j] = v0[j]; x[VEC + j] = v1[j]; }
                map_batch<2 * VEC>(x, y, xf);
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    if (h == 1 && !second) break;
                    Acc* to = mapped + (i + h * 256) * VEC;
#pragma unroll
                    for (int j0 = 0; j0 < VEC; j0 += AV) {
                        VA w;
#pragma unroll
                        for (int j = 0; j < AV; ++j) w[j] = y[h * VEC + j0 + j];
                        *(VA*)(to + j0) = w;
                    }
                }
            }
            for (int e = nv * VEC + t; e < ne; e += 256) mapped[e] = xf(p[e], (Pos)0);
        }
    } else {
        for (int i = t; i < nv; i += 256) {
            if constexpr (VEC == 1) lds[i] = p[i];
            else ((V*)lds)[i] = load_nt((const V*)p + i);
        }
        for (int e = nv * VEC + t; e < ne; e += 256) lds[e] = p[e];             // fewer than VEC elements
    }
    __syncthreads();
    const int tpl = 1 << tpl_log2;                       // <= 16 and <= m
    const int nl = ns * inner;
    const int items = nl << tpl_log2;
    for (int base = 0; base < items; base += 256) {      // uniform trip count: the DPP fold below needs every lane
        const int idx = base + t;
        const int l = idx >> tpl_log2, part = idx & (tpl - 1);
        Acc acc = Op::template identity<Acc>();
        if (l < nl) {
            const int sl = l / inner;
            const In* line = lds + sl * slab + (l - sl * inner);
            const Acc* mapped_line = (const Acc*)lds_raw + sl * slab + (l - sl * inner);
            const int count = (m - part + tpl - 1) >> tpl_log2;          // elements k = part (mod tpl) of 0 .. m-1
            int k = part + ((sl * (tpl - m)) & rot_mask);                 // < tpl + P <= 2 m
            if (k >= m) k -= m;
            for (int c = 0; c < count; ++c) {
                if constexpr (MAPPED_IN_LDS) acc = op(acc, mapped_line[k * inner]);
                else acc = op(acc, xf(line[k * inner], (Pos)k));
                k += tpl;
                if (k >= m) k -= m;
            }
        }
        if (tpl_log2 >= 1) acc = op(acc, dpp_move<DPP_QUAD_XOR1>(acc, acc));
        if (tpl_log2 >= 2) acc = op(acc, dpp_move<DPP_QUAD_XOR2>(acc, acc));
        if (tpl_log2 >= 3) acc = op(acc, dpp_move<DPP_ROW_HALF_MIRROR>(acc, acc));
        if (tpl_log2 >= 4) acc = op(acc, dpp_move<DPP_ROW_MIRROR>(acc, acc));
        if (l < nl && part == 0) sink(slab0 * inner + l, acc);
    }
}

// ---- completion count of the workgroups that share a result ----------------------------------------------------------
// Called by one thread after the workgroup's partials are at the coherent level; true for the last of the `n` workgroups
// of `slot`.  Atomics on one address complete one after the other, and hundreds of workgroups that finish together
// queue up behind one ticket (findmax(A; dims=2) of 64 x 500_000 Float32, one strip, 512 workgroups: 72 us; the same
// data as 64 x 7812 x 64, sixty-four tickets: 25 us).  With groups > 1 the workgroups take a ticket of their group of
// TICKET_GROUP first and only the last of a group takes the slot's own: slot * (groups + 1) + group, then + groups.
// The group tickets are left at zero; the caller clears the slot's own when it is done (arrival_reset).
__device__ __forceinline__ bool last_arrival(uint32_t* tickets, int64_t slot, int idx, int n, int groups) {
    if (groups <= 1) {
        const uint32_t old = __hip_atomic_fetch_add(&tickets[slot * TICKET_STRIDE], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return old == (uint32_t)n - 1u;
    }
    uint32_t* base = tickets + slot * (groups + 1) * TICKET_STRIDE;
    const int grp = idx / TICKET_GROUP;
    const int gsize = grp == groups - 1 ? n - grp * TICKET_GROUP : TICKET_GROUP;
    const uint32_t old = __hip_atomic_fetch_add(&base[grp * TICKET_STRIDE], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (old != (uint32_t)gsize - 1u) return false;
    __hip_atomic_store(&base[grp * TICKET_STRIDE], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t top = __hip_atomic_fetch_add(&base[groups * TICKET_STRIDE], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return top == (uint32_t)groups - 1u;
}
__device__ __forceinline__ void arrival_reset(uint32_t* tickets, int64_t slot, int groups) {
    if (groups <= 1) tickets[slot * TICKET_STRIDE] = 0;
    else tickets[(slot * (groups + 1) + groups) * TICKET_STRIDE] = 0;
}
// groups for last_arrival: two levels when more than two groups' worth of workgroups share a slot and the tickets suffice
inline int arrival_groups(int64_t slots, int64_t n) {
    const int64_t groups = (n + TICKET_GROUP - 1) / TICKET_GROUP;
    return (groups > 2 && slots * (groups + 1) <= (int64_t)WS_TICKET_COUNT) ? (int)groups : 1;
}

// ---- 1 < inner < 64 with long lines: contiguous runs of whole rows ---------------------------------------
// (sum(A; dims=2) of a 3 x 1_000_000 array, perf/array.jl:91,96; the fold over the long dim of a 2 x 3 x N array.)
// A wave per line reads one element in `inner`, a quarter or less of every cache line at a time.  Here thread t of
// the inner * R threads (R = 256 / inner whole rows) reads element t of the workgroup's current run of R rows:
// consecutive lanes, consecutive addresses, and because a pass advances by whole rows the thread's column t % inner
// never changes.  The R threads of a column meet in LDS.  grid (msplits, outer): a workgroup takes rows_per_split
// rows of one slab; partials[(o * msplits + ms) * inner + column], one ticket per slab, the last arrival folds.
template <typename In, typename Acc, typename Xf, typename Op, typename Sink>
__global__ __launch_bounds__(256) void reduce_narrow_kernel(const In* __restrict__ A, LineGeom g, Xf xf, Op op, Sink sink,
                                                            Acc* partials, uint32_t* tickets, int64_t rows_per_split, int tgroups) {
    typedef typename Xf::Pos Pos;
    __shared__ Acc lds[256];
    __shared__ int is_last;
    const int t = threadIdx.x;
    const int inner = (int)g.inner;
    const int R = 256 / inner, T = R * inner;
    const int ms = blockIdx.x, msplits = gridDim.x;
    const int64_t o = blockIdx.y;
    const int64_t r0 = (int64_t)ms * rows_per_split;
    int64_t r1 = r0 + rows_per_split;
    if (r1 > g.mid) r1 = g.mid;
    const In* slab = A + o * g.inner * g.mid;
    constexpr int NU = 8;                  // loads in flight per thread
    Acc acc[NU];
#pragma unroll
    for (int u = 0; u < NU; ++u) acc[u] = Op::template identity<Acc>();
    if (t < T) {
        const int rt = t / inner;
        int64_t row = r0 + rt;
        const In* p = slab + r0 * inner + t;       // = slab + row * inner + column; a pass advances by T elements
        for (; row + (NU - 1) * R < r1; row += NU * R, p += NU * T) {
            In v[NU];
#pragma unroll
            for (int u = 0; u < NU; ++u) v[u] = p[u * T];
#pragma unroll
            for (int u = 0; u < NU; ++u) acc[u] = acc_step(op, acc[u], xf(v[u], (Pos)(row + u * R)));
        }
        for (; row < r1; row += R, p += T) acc[0] = acc_step(op, acc[0], xf(p[0], (Pos)row));
    }
    Acc all = acc[0];
#pragma unroll
    for (int u = 1; u < NU; ++u) all = op(all, acc[u]);
    lds[t] = all;
    __syncthreads();
    Acc r = Op::template identity<Acc>();
    if (t < inner)
        for (int k = 0; k < R; ++k) r = op(r, lds[t + k * inner]);
    if (msplits == 1) {
        if (t < inner) sink(t + o * g.inner, r);
        return;
    }
    if (t < inner) {
        store_agent(&partials[(o * msplits + ms) * inner + t], r);
        publish_barrier();
    }
    __syncthreads();   // every partial of this workgroup is at the coherent level before the ticket moves
    if (t == 0) is_last = last_arrival(tickets, o, ms, msplits, tgroups);
    __syncthreads();
    if (!is_last) return;
    // the last arrival folds the msplits rows of partials the way it folded its own rows: thread t takes column
    // t % inner of rows t / inner, t / inner + R, ...; the R threads of a column meet in LDS
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    Acc f = Op::template identity<Acc>();
    if (t < T) {
        // (eight independent loads at a time: one after the other, each waits for the one before -- msplits / R round trips)
        const int rt = t / inner, c = t - rt * inner;
        const Acc* pc = partials + o * msplits * inner + c;
        int i = rt;
        for (; i + 7 * R < msplits; i += 8 * R) {
            Acc v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = pc[(int64_t)(i + u * R) * inner];
#pragma unroll
            for (int u = 0; u < 8; ++u) f = op(f, v[u]);
        }
        for (; i < msplits; i += R) f = op(f, pc[(int64_t)i * inner]);
    }
    __syncthreads();     // lds is free again
    lds[t] = f;
    __syncthreads();
    if (t < inner) {
        Acc r2 = Op::template identity<Acc>();
        for (int k = 0; k < R; ++k) r2 = op(r2, lds[t + k * inner]);
        sink(t + o * g.inner, r2);
    }
    if (t == 0) arrival_reset(tickets, o, tgroups);
}

// ---- inner >= 64: lanes along `inner` -------------------------------------------------------------
// grid (strips * outer, msplits): the outer index shares the x axis with the strips (the y and z axes of a grid end
// at 65535, and a 64 x 2 x 70000 array has that many outer indices and more); workgroup = 4 waves; a wave owns
// 64 * VEC adjacent columns of a strip and every 4th row of the row batches dealt to its workgroup.
// PACKED (one strip whose rows fill at most half of it, element-aligned vectors): P = ceil(inner / VEC) lanes hold a row
// and a load instruction takes Q = 64 / P consecutive rows; lane group q sees the rows q, q + Q, ... of what the wave
// is dealt, and the groups are folded across the lanes at the end.  (findmax(A; dims=2) of a 64 x 500_000 Float32
// array: 16 of 64 lanes busy, 105 us; sums of such arrays are viewed as wider ones by the host instead.)
template <typename T> __device__ __forceinline__ T shfl_down_words(const T& v, int delta) {
    static_assert(sizeof(T) % 4 == 0, "whole words");
    uint32_t w[sizeof(T) / 4];
    __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
    for (unsigned i = 0; i < sizeof(T) / 4; ++i) w[i] = (uint32_t)__shfl_down((int)w[i], delta, WAVE);
    T r;
    __builtin_memcpy(&r, w, sizeof(T));
    return r;
}

template <typename In, typename Acc, typename Xf, typename Op, typename Sink, bool VECTOR, int UNROLL, bool PACKED = false>
__global__ __launch_bounds__(256) void reduce_strided_kernel(const In* __restrict__ A, LineGeom g, Xf xf, Op op, Sink sink,
                                                             Acc* partials, uint32_t* tickets, int strips, int tgroups, int P = WAVE) {
    constexpr int VEC = VECTOR ? 16 / sizeof(In) : 1;
    constexpr int COLS = WAVE * VEC;   // columns per strip
    constexpr int NW = 4;
    typedef typename VecOf<In, VEC>::type V;
    __shared__ Acc lds[NW][COLS];
    __shared__ int is_last;
    const int ms = blockIdx.y, msplits = gridDim.y;
    const int64_t tile = blockIdx.x;                    // o * strips + strip
    const int64_t o = tile / strips;
    const int strip = (int)(tile - o * strips);
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int Q = PACKED ? WAVE / P : 1;                // rows per load instruction
    const int q = PACKED ? lane / P : 0;                // this lane's row among them
    const int pl = PACKED ? lane - q * P : lane;        // this lane's vector within the row
    const int64_t nominal = (int64_t)strip * COLS + (int64_t)pl * VEC;
    const bool live = nominal < g.inner && q < Q;
    // 4- and 8-byte elements: vectors at any element-aligned address (load_nt_elems), so rows need be no whole number
    // of vectors.  The last vector of such a row starts VEC elements before the row's end instead of running into the
    // next row; the `dup` leading columns it shares with the lane before are dropped after the loop.
    constexpr bool ANY_ALIGN = VECTOR && sizeof(In) >= 4;
    const int64_t col0 = (ANY_ALIGN && live && nominal + VEC > g.inner) ? g.inner - VEC : nominal;
    const int dup = (int)(nominal - col0);
    const int64_t slab = o * g.inner * g.mid;
    auto load_row = [](const In* q) -> V {
        if constexpr (ANY_ALIGN) return load_nt_elems<In, VEC>(q);
        else return load_nt((const V*)q);
    };

    Acc acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = Op::template identity<Acc>();
    // Rows are dealt out in batches of UNROLL * 4: batch b goes to workgroup b % msplits, so at any moment the
    // workgroups of a strip (and, strip by strip, the whole grid) read one compact band of rows.  Giving every
    // workgroup one long contiguous slice instead spreads the reads over rows megabytes apart, which the
    // memory system serves up to 20 % slower when the row pitch is a power of two.
    // (PACKED: what is dealt out are groups of Q consecutive rows; `m` counts groups, the lane's row is m * Q + q)
    constexpr int64_t BATCH = (int64_t)UNROLL * NW;
    const int64_t ngroups = PACKED ? (g.mid + Q - 1) / Q : g.mid;
    const int64_t nbatches = (ngroups + BATCH - 1) / BATCH;
    if (live) {
        const In* p = A + slab + col0 + (PACKED ? (int64_t)q * g.inner : 0);
        const int64_t pitch = PACKED ? g.inner * Q : g.inner;
        for (int64_t b = ms; b < nbatches; b += msplits) {
            const int64_t m = b * BATCH + wave;
            V v[UNROLL];
            if (PACKED ? (m + (UNROLL - 1) * NW) * Q + (Q - 1) < g.mid : m + (UNROLL - 1) * NW < g.mid) {
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) v[u] = load_row(p + (m + u * NW) * pitch);
                if constexpr (XfIsBatch<Xf>::value) {
                    In x[UNROLL * VEC];
                    Acc y[UNROLL * VEC];
#pragma unroll
                    for (int u = 0; u < UNROLL; ++u) {
                        if constexpr (VEC == 1) x[u] = v[u];
                        else {
#pragma unroll
                            for (int j = 0; j < VEC; ++j) x[u * VEC + j] = v[u][j];
                        }
                    }
                    map_batch<UNROLL * VEC>(x, y, xf);
#pragma unroll
                    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
                        for (int j = 0; j < VEC; ++j) acc[j] = acc_step(op, acc[j], y[u * VEC + j]);
                } else {
#pragma unroll
                    for (int u = 0; u < UNROLL; ++u) {
                        const typename Xf::Pos e0 = (typename Xf::Pos)(PACKED ? (m + u * NW) * Q + q : m + u * NW);
                        if constexpr (VEC == 1) acc[0] = acc_step(op, acc[0], xf(v[u], e0));
                        else {
#pragma unroll
                            for (int j = 0; j < VEC; ++j) acc[j] = acc_step(op, acc[j], xf(v[u][j], e0));
                        }
                    }
                }
            } else {
                for (int64_t r = m; (PACKED ? r * Q + q : r) < g.mid; r += NW) {
                    const V x = load_row(p + r * pitch);
                    const typename Xf::Pos e0 = (typename Xf::Pos)(PACKED ? r * Q + q : r);
                    if constexpr (VEC == 1) acc[0] = acc_step(op, acc[0], xf(x, e0));
                    else {
#pragma unroll
                        for (int j = 0; j < VEC; ++j) acc[j] = acc_step(op, acc[j], xf(x[j], e0));
                    }
                }
            }
        }
    }
    if constexpr (PACKED) {
        // the lane groups of a wave, folded into group 0 (idle lanes hold the identity; a lane past the wave's end has no partner)
        for (int delta = P; delta < WAVE; delta <<= 1) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const Acc y = shfl_down_words(acc[j], delta);
                if (lane + delta < WAVE) acc[j] = op(acc[j], y);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        if (j >= dup && q == 0) lds[wave][pl * VEC + j - dup] = acc[j];      // columns past the row's end keep whatever LDS held: never sunk
    __syncthreads();
    // thread t folds columns t, t + 256, ... of the strip: a strip has 64 * VEC columns -- 256 for 4-byte elements, one
    // a thread; 512 or 1024 for 2- and 1-byte elements
    const int t = threadIdx.x;
    constexpr int CPT = (COLS + 255) / 256;              // columns per thread
    Acc r[CPT];
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
        const int tc = t + c * 256;
        r[c] = Op::template identity<Acc>();
        if (tc < COLS) {
            r[c] = lds[0][tc];
#pragma unroll
            for (int w = 1; w < NW; ++w) r[c] = op(r[c], lds[w][tc]);
        }
    }
    if (msplits == 1) {
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            const int tc = t + c * 256;
            const int64_t col = (int64_t)strip * COLS + tc;
            if (tc < COLS && col < g.inner) sink(col + o * g.inner, r[c]);
        }
        return;
    }
    // partials[(o * strips + strip) * msplits + ms][COLS]
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
        const int tc = t + c * 256;
        if (tc < COLS && (int64_t)strip * COLS + tc < g.inner) store_agent(&partials[(tile * msplits + ms) * COLS + tc], r[c]);
    }
    publish_barrier();
    __syncthreads();   // every partial of this workgroup is at the coherent level before the ticket moves
    // Fold of `nrows` rows of partials ([row][COLS]) by this workgroup: wave w folds rows w, w + 4, ... for the columns it
    // streamed, thread t then joins the four waves for its columns; fixed order.  The rows were written through to the
    // coherent level; one acquire (cache invalidate) lets the workgroup read them with plain, batched loads.  Lanes whose
    // columns lie past the row's end read nothing.
    auto fold_rows = [&](const Acc* rows, int nrows, Acc (&out)[CPT]) {
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        const Acc* prow = rows + lane * VEC;
        Acc f[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) f[j] = Op::template identity<Acc>();
        const bool fold_live = (int64_t)strip * COLS + (int64_t)lane * VEC < g.inner;
        int i = fold_live ? wave : nrows;
        if constexpr (VEC <= 4) {
            constexpr int FU = 4;            // rows a wave has in flight (8: registers 64 -> 96 for findmax, and the many small workgroups of a short reduced dim lose occupancy)
            for (; i + (FU - 1) * NW < nrows; i += FU * NW) {
                Acc v[FU][VEC];
#pragma unroll
                for (int u = 0; u < FU; ++u)
#pragma unroll
                    for (int j = 0; j < VEC; ++j) v[u][j] = prow[(int64_t)(i + u * NW) * COLS + j];
#pragma unroll
                for (int u = 0; u < FU; ++u)
#pragma unroll
                    for (int j = 0; j < VEC; ++j) f[j] = op(f[j], v[u][j]);
            }
        }
        for (; i < nrows; i += NW)
#pragma unroll
            for (int j = 0; j < VEC; ++j) f[j] = op(f[j], prow[(int64_t)i * COLS + j]);
        __syncthreads();     // lds is free again
#pragma unroll
        for (int j = 0; j < VEC; ++j) lds[wave][lane * VEC + j] = f[j];
        __syncthreads();
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            const int tc = t + c * 256;
            out[c] = Op::template identity<Acc>();
            if (tc < COLS) {
                out[c] = lds[0][tc];
#pragma unroll
                for (int w = 1; w < NW; ++w) out[c] = op(out[c], lds[w][tc]);
            }
        }
    };
    Acc res[CPT];
    if (tgroups > 1) {
        // Two levels (see last_arrival): the last arrival of a group of TICKET_GROUP workgroups folds the group's rows into
        // one row of group partials, behind the partials of all tiles, and only then takes the strip's own ticket; the last
        // group folds the group rows.  One workgroup folding all 512 rows of a single strip took 45 of the kernel's 70 us
        // (findmax(A; dims=2), 64 x 500_000 Float32), whatever the loads in flight: the groups fold side by side.
        const int grp = ms / TICKET_GROUP;
        const int gsize = grp == tgroups - 1 ? msplits - grp * TICKET_GROUP : TICKET_GROUP;
        uint32_t* base = tickets + tile * (tgroups + 1) * TICKET_STRIDE;
        if (t == 0) {
            const uint32_t old = __hip_atomic_fetch_add(&base[grp * TICKET_STRIDE], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            is_last = (old == (uint32_t)gsize - 1u);
        }
        __syncthreads();
        if (!is_last) return;
        fold_rows(partials + (tile * msplits + (int64_t)grp * TICKET_GROUP) * COLS, gsize, res);
        Acc* gpartials = partials + (int64_t)gridDim.x * msplits * COLS;
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            const int tc = t + c * 256;
            if (tc < COLS && (int64_t)strip * COLS + tc < g.inner) store_agent(&gpartials[(tile * tgroups + grp) * COLS + tc], res[c]);
        }
        publish_barrier();
        __syncthreads();   // (also: everybody has read is_last before it is written again)
        if (t == 0) {
            __hip_atomic_store(&base[grp * TICKET_STRIDE], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t top = __hip_atomic_fetch_add(&base[tgroups * TICKET_STRIDE], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            is_last = (top == (uint32_t)tgroups - 1u);
        }
        __syncthreads();
        if (!is_last) return;
        fold_rows(gpartials + tile * tgroups * COLS, tgroups, res);
    } else {
        if (t == 0) is_last = last_arrival(tickets, tile, ms, msplits, 1);
        __syncthreads();
        if (!is_last) return;
        fold_rows(partials + tile * msplits * COLS, msplits, res);     // last arrival of the strip: all its rows
    }
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
        const int tc = t + c * 256;
        const int64_t col = (int64_t)strip * COLS + tc;
        if (tc < COLS && col < g.inner) sink(col + o * g.inner, res[c]);
    }
    if (t == 0) arrival_reset(tickets, tile, tgroups);
}

// ---- arbitrary masks: one wave per output ------------------------------------------------------------
struct GenericGeom {
    int     nkeep, nred;
    int64_t keep_size[RK_MAX_DIMS], keep_stride[RK_MAX_DIMS];
    int64_t red_size[RK_MAX_DIMS], red_stride[RK_MAX_DIMS];
    int64_t nout, nred_total;
};

// GROUP lanes share an output: 1 (a handful of elements per output and many outputs: maximum(A; dims=(1, 3)) of a
// 4 x 1_000_000 x 4 array -- a wave per output would idle 48 lanes and there are a million outputs), 64, or the whole
// workgroup (few outputs with many elements each: findmax(A; dims=(1, 3)) of a 256^3 array has 256 outputs).
// I is the type the index of a reduced element is split in: 32-bit division is several times cheaper than 64-bit.
template <typename In, typename Acc, typename Xf, typename Op, typename Sink, int BLOCK, int GROUP, typename I>
__global__ __launch_bounds__(BLOCK) void reduce_generic_kernel(const In* __restrict__ A, GenericGeom g, Xf xf, Op op, Sink sink) {
    __shared__ Acc lds[BLOCK / WAVE];
    const int64_t q = GROUP == BLOCK ? (int64_t)blockIdx.x : ((int64_t)blockIdx.x * BLOCK + threadIdx.x) / GROUP;
    if (q >= g.nout) return;                 // uniform over the lanes that share an output
    int64_t base = 0, rem = q;
    for (int d = 0; d < g.nkeep; ++d) {
        base += (rem % g.keep_size[d]) * g.keep_stride[d];
        rem /= g.keep_size[d];
    }
    Acc a = Op::template identity<Acc>();
    const I total = (I)g.nred_total;
    // NU elements a round, their loads issued together (few outputs mean few waves: 256 workgroups for findmax(A; dims=(1, 3))
    // of a 256^3 array, and one load in flight per lane leaves the memory system idle)
    constexpr int NU = GROUP == 1 ? 1 : 4;
    for (I k = (I)(threadIdx.x % GROUP); k < total; k += (I)(NU * GROUP)) {       // total < 2^31 when I has 32 bits: no wrap
        int64_t off[NU];
        In v[NU];
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            I r = k + (I)(u * GROUP);
            off[u] = -1;
            if (r < total) {
                off[u] = base;
                for (int d = 0; d < g.nred; ++d) {
                    const I n = (I)g.red_size[d];
                    const I c = d == g.nred - 1 ? r : r % n;
                    off[u] += (int64_t)c * g.red_stride[d];
                    r /= n;
                }
                v[u] = A[off[u]];
            }
        }
#pragma unroll
        for (int u = 0; u < NU; ++u)
            if (off[u] >= 0) a = op(a, xf(v[u], (typename Xf::Pos)off[u]));
    }
    if constexpr (GROUP == BLOCK) a = block_reduce<BLOCK / WAVE>(a, op, lds);
    else if constexpr (GROUP == WAVE) a = wave_reduce(a, op);
    if (threadIdx.x % GROUP == 0) sink(q, a);
}

// ---- host side: pick a kernel and launch -------------------------------------------------------------
struct ReducePlan {
    enum Kind { SPLIT, WAVE_LINES, THREAD_LINES, SHORT_LINES, STRIDED, NARROW, GENERIC, COLS } kind;
    bool    vector;
    int     splits;      // SPLIT: workgroups per line; STRIDED, NARROW: slices of mid
    int64_t rows_per_split;   // NARROW
    int     strips;      // STRIDED
    int     slabs_per_block, tpl_log2, rot_mask;      // SHORT_LINES
    size_t  payload;     // bytes of partials
};

// Tunables (workgroups per compute unit the streaming kernels aim for).
int tune_reduce_blocks_per_cu();           // rk_api.hip
int tune_reduce_strided_blocks_per_cu();   // rk_api.hip
int tune_reduce_wave_max_bytes();          // rk_api.hip

template <typename In, typename Acc>
inline ReducePlan plan_reduce(const void* A, const Shape3& s, bool single_run, size_t cap = WS_PARTIALS_BYTES, int grid_scale = 1,
                              int short_lines_tile = 16384 / (int)sizeof(In), bool cols_ok = false) {
    ReducePlan p{};
    const int cus = device_info().cus;
    const int64_t target_blocks = (int64_t)cus * tune_reduce_blocks_per_cu() * grid_scale;
    constexpr int VEC = 16 / sizeof(In);
    if (!single_run) { p.kind = ReducePlan::GENERIC; return p; }
    const int64_t nlines = s.inner * s.outer;
    const int64_t slab = s.inner * s.mid;
    // (rows of 64 elements or more that are whole vectors stream as well through the strided kernel)
    if (s.mid >= 2 && nlines >= 1024 && slab <= short_lines_tile && (s.inner > 1 || s.mid <= SHORT_LINES_MAX) &&
        (s.inner < 64 || s.inner % VEC != 0 || !is_aligned(A, 16))) {
        // whole slabs per block, and (for the vector loads) a block size in bytes that is a multiple of 16
        int spb = short_lines_tile / (int)slab;
        bool vector = is_aligned(A, 16);
        if (vector) {
            int q = 16;                                                      // 16 / gcd(slab bytes, 16)
            for (size_t bytes = (size_t)slab * sizeof(In); q > 1 && bytes % 2 == 0; bytes /= 2) q /= 2;
            if (spb / q > 0) spb -= spb % q;
            else vector = false;
        }
        const int lines = spb * (int)s.inner;
        int tl = 0;
        while (tl < 4 && (lines << tl) < 256 && (2 << tl) <= s.mid) ++tl;
        if ((lines << tl) >= 128) {                                          // else too few lanes would fold
            int pow2 = 1;
            while (pow2 * 2 <= s.mid && pow2 < 64) pow2 *= 2;
            p.kind = ReducePlan::SHORT_LINES;
            p.vector = vector;
            p.slabs_per_block = spb;
            p.tpl_log2 = tl;
            p.rot_mask = pow2 - 1;
            return p;
        }
    }
    if (cols_ok && s.inner >= 64 && s.mid <= 16 && nlines >= 4096 && is_aligned(A, sizeof(In))) { p.kind = ReducePlan::COLS; return p; }
    if (s.inner >= 64) {
        p.kind = ReducePlan::STRIDED;
        // 4- and 8-byte elements: vectors at any element-aligned address, rows of any length >= a vector
        p.vector = sizeof(In) >= 4 ? is_aligned(A, sizeof(In)) : (s.inner % VEC == 0) && is_aligned(A, 16);
        const int cols = WAVE * (p.vector ? VEC : 1);
        const int64_t strips = (s.inner + cols - 1) / cols;
        p.strips = (int)strips;
        int64_t tiles = strips * s.outer;
        int64_t ms = 1;
        // Few, deep workgroups win here: each lane keeps 4 x 16 B in flight, and every extra share of
        // `mid` costs a row of partials plus a longer fold.
        const int64_t strided_target = (int64_t)cus * tune_reduce_strided_blocks_per_cu() * grid_scale;
        if (tiles < strided_target && tiles <= (int64_t)WS_TICKET_COUNT) {
            ms = (strided_target + tiles - 1) / tiles;
            const int64_t max_ms = (s.mid + 31) / 32;      // at least 32 rows per workgroup
            if (ms > max_ms) ms = max_ms;
            if (ms > 1024) ms = 1024;
            const int64_t fit = (int64_t)(cap / sizeof(Acc)) / (tiles * cols);
            if (ms > fit) ms = fit;
            if (ms < 1) ms = 1;
        }
        p.splits = (int)ms;
        p.payload = ms > 1 ? (size_t)(tiles * ms * cols) * sizeof(Acc) : 0;
        return p;
    }
    if (s.mid <= 16 && nlines >= 4096) { p.kind = ReducePlan::THREAD_LINES; return p; }
    // (from 64 rows on: below 1024 rows and above the 16 KiB slabs of the LDS kernel the alternative is a wave per line
    // that reads one element in `inner` -- sum(A; dims=2) of 33 x 1000 x 1000 Float32: 0.8 TB/s)
    if (s.inner > 1 && s.mid >= 64 && s.outer <= 65535 && s.outer <= (int64_t)WS_TICKET_COUNT) {
        p.kind = ReducePlan::NARROW;
        const int64_t rows_per_pass = 256 / s.inner;
        // every extra workgroup costs a row of partials and a longer fold: two per compute unit measured best
        // (63 x 1048576 Float32: 1024 workgroups 107 us, 512 73 us), each with at least 16 passes of its own
        int64_t want = (target_blocks + s.outer - 1) / s.outer;
        const int64_t max_splits = (s.mid + 16 * rows_per_pass - 1) / (16 * rows_per_pass);
        if (want > max_splits) want = max_splits;
        if (want > 4096) want = 4096;
        const int64_t fit = (int64_t)(cap / sizeof(Acc)) / (s.outer * s.inner);
        if (want > fit) want = fit;
        if (want < 1) want = 1;
        p.splits = (int)want;
        p.rows_per_split = (s.mid + want - 1) / want;
        p.payload = want > 1 ? (size_t)(s.outer * want * s.inner) * sizeof(Acc) : 0;
        return p;
    }
    const bool contiguous = (s.inner == 1);
    // Plenty of lines: a wave per line fills every compute unit -- but only for short lines.  With a wave per
    // 32 KiB line all 8192 resident waves stream different DRAM pages at once; a workgroup per line keeps the
    // active region contiguous (measured on 8192 x 8192 Float32: 6.4 -> 6.65 TB/s, findmax 5.7 -> 6.2 TB/s).
    if (nlines >= (int64_t)cus * 16 &&
        (s.mid * (int64_t)sizeof(In) <= tune_reduce_wave_max_bytes() || nlines > 65535)) {
        p.kind = ReducePlan::WAVE_LINES;
        p.vector = contiguous && s.mid >= 2 * VEC;
        return p;
    }
    p.kind = ReducePlan::SPLIT;
    p.vector = contiguous && s.mid >= 2 * VEC;
    // a workgroup pass covers 256 lanes * 16 B * 4 loads = 16 KiB; give each split >= 2 passes
    const int64_t per_pass = 256 * (p.vector ? VEC : 1) * 4;
    int64_t want = (target_blocks + nlines - 1) / nlines;
    int64_t max_splits = (s.mid + 2 * per_pass - 1) / (2 * per_pass);
    if (want > max_splits) want = max_splits;
    if (want > 4096) want = 4096;
    const int64_t fit = (int64_t)(cap / sizeof(Acc)) / (2 * nlines);   // partials + group partials
    if (want > fit) want = fit;
    const int64_t groups = (want + TICKET_GROUP - 1) / TICKET_GROUP;
    if (want < 1 || nlines * (groups + 1) > (int64_t)WS_TICKET_COUNT) want = 1;
    p.splits = (int)want;
    p.payload = want > 1 ? (size_t)(nlines * (want + groups)) * sizeof(Acc) : 0;
    return p;
}

template <typename In, typename Acc, typename Xf, typename Op, typename Sink>
inline int32_t launch_reduce(const In* A, int ndim, const int64_t* shape, uint32_t mask, Xf xf, Op op, Sink sink,
                             void* ws, size_t ws_bytes, hipStream_t stream, size_t cap = WS_PARTIALS_BYTES) {
    const Shape3 s = collapse3(ndim, shape, mask);
    // A program for f costs scalar branches per token and wave: more resident waves hide them better
    // (2^26 Float32, x -> x + 1: 3.4 -> 5.2 TB/s with twice the workgroups; 9 tokens: 2.3 -> 2.6 TB/s with four times)
    int grid_scale = 1;
    if constexpr (XfIsBatch<Xf>::value) grid_scale = xf.n_tokens > 4 ? 4 : 2;
    // reduce_cols_kernel: 4- and 8-byte elements, f applied per element (not a traced program); not findmax / findmin,
    // whose outputs (a value and ndims indices each, more bytes than the input when the reduced extent is 3) want a lane
    // per output: 200 x 3 x 50000 Float32 dims=2 1.0 TB/s of input from the strided kernel, 0.43 from this one
    constexpr bool COLS_OK = sizeof(In) >= 4 && !XfIsBatch<Xf>::value && !XfIsArg<Xf>::value;
    const ReducePlan p = plan_reduce<In, Acc>(A, s, s.single_run, cap, grid_scale, ShortLinesTile<In, Acc, Xf>::ELEMS, COLS_OK);
    Workspace w{};
    if (p.payload > cap) return RK_ERR_WORKSPACE;   // the planner never asks for more
    if (p.payload > 0 && !carve_workspace(ws, ws_bytes, 0, &w)) return RK_ERR_WORKSPACE;
    LineGeom g{s.inner, s.mid, s.inner * s.outer};
    constexpr int UNROLL = sizeof(In) >= 4 ? 4 : 2;
    switch (p.kind) {
        case ReducePlan::SPLIT: {
            if (g.nlines > 65535) return RK_ERR_TOO_LARGE;
            dim3 grid(p.splits, (unsigned)g.nlines);
            if (p.vector)
                reduce_split_kernel<In, Acc, Xf, Op, Sink, true, 256, UNROLL><<<grid, 256, 0, stream>>>(A, g, xf, op, sink, (Acc*)w.partials, w.tickets);
            else
                reduce_split_kernel<In, Acc, Xf, Op, Sink, false, 256, UNROLL><<<grid, 256, 0, stream>>>(A, g, xf, op, sink, (Acc*)w.partials, w.tickets);
            break;
        }
        case ReducePlan::WAVE_LINES: {
            const int64_t blocks = (g.nlines + 3) / 4;
            if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
            if (p.vector)
                reduce_wave_kernel<In, Acc, Xf, Op, Sink, true, 256, UNROLL><<<(unsigned)blocks, 256, 0, stream>>>(A, g, xf, op, sink);
            else
                reduce_wave_kernel<In, Acc, Xf, Op, Sink, false, 256, UNROLL><<<(unsigned)blocks, 256, 0, stream>>>(A, g, xf, op, sink);
            break;
        }
        case ReducePlan::COLS: {
            if constexpr (COLS_OK) {
                constexpr int64_t VEC = 16 / (int64_t)sizeof(In);
                const int64_t groups_per_row = (s.inner + VEC - 1) / VEC;
                if (groups_per_row > INT64_MAX / (s.outer > 0 ? s.outer : 1)) return RK_ERR_TOO_LARGE;
                const int64_t ngroups = groups_per_row * s.outer, blocks = (ngroups + 255) / 256;
                if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
                reduce_cols_kernel<In, Acc, Xf, Op, Sink><<<(unsigned)blocks, 256, 0, stream>>>(A, g, xf, op, sink, groups_per_row, ngroups);
            }
            break;
        }
        case ReducePlan::THREAD_LINES: {
            const int64_t blocks = (g.nlines + 255) / 256;
            if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
            reduce_thread_kernel<In, Acc, Xf, Op, Sink, 256><<<(unsigned)blocks, 256, 0, stream>>>(A, g, xf, op, sink);
            break;
        }
        case ReducePlan::SHORT_LINES: {
            const int64_t blocks = (s.outer + p.slabs_per_block - 1) / p.slabs_per_block;
            if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
            if (p.vector)
                reduce_short_lines_kernel<In, Acc, Xf, Op, Sink, true><<<(unsigned)blocks, 256, 0, stream>>>(
                    A, (int)s.inner, (int)s.mid, s.outer, p.slabs_per_block, p.tpl_log2, p.rot_mask, xf, op, sink);
            else
                reduce_short_lines_kernel<In, Acc, Xf, Op, Sink, false><<<(unsigned)blocks, 256, 0, stream>>>(
                    A, (int)s.inner, (int)s.mid, s.outer, p.slabs_per_block, p.tpl_log2, p.rot_mask, xf, op, sink);
            break;
        }
        case ReducePlan::STRIDED: {
            const int64_t tiles = (int64_t)p.strips * s.outer;
            if (tiles > 0x7fffffff) return RK_ERR_TOO_LARGE;
            dim3 grid((unsigned)tiles, p.splits);
            int tgroups = arrival_groups(tiles, p.splits);
            // the group rows lie behind the partials: one level where they do not fit
            if (tgroups > 1 && (size_t)(tiles * (p.splits + tgroups)) * (WAVE * (p.vector ? 16 / sizeof(In) : 1)) * sizeof(Acc) > cap) tgroups = 1;
            if constexpr (XfIsArg<Xf>::value && sizeof(In) >= 4) {
                constexpr int VEC = 16 / (int)sizeof(In);
                if (p.vector && p.strips == 1 && s.inner >= VEC && s.inner * 2 <= WAVE * VEC) {
                    reduce_strided_kernel<In, Acc, Xf, Op, Sink, true, UNROLL, true><<<grid, 256, 0, stream>>>(
                        A, g, xf, op, sink, (Acc*)w.partials, w.tickets, p.strips, tgroups, (int)((s.inner + VEC - 1) / VEC));
                    break;
                }
            }
            if (p.vector)
                reduce_strided_kernel<In, Acc, Xf, Op, Sink, true, UNROLL><<<grid, 256, 0, stream>>>(A, g, xf, op, sink, (Acc*)w.partials, w.tickets, p.strips, tgroups);
            else
                reduce_strided_kernel<In, Acc, Xf, Op, Sink, false, UNROLL><<<grid, 256, 0, stream>>>(A, g, xf, op, sink, (Acc*)w.partials, w.tickets, p.strips, tgroups);
            break;
        }
        case ReducePlan::NARROW: {
            dim3 grid(p.splits, (unsigned)s.outer);
            reduce_narrow_kernel<In, Acc, Xf, Op, Sink><<<grid, 256, 0, stream>>>(A, g, xf, op, sink, (Acc*)w.partials, w.tickets, p.rows_per_split,
                                                                                  arrival_groups(s.outer, p.splits));
            break;
        }
        case ReducePlan::GENERIC: {
            GenericGeom gg{};
            int64_t stride = 1;
            gg.nout = 1; gg.nred_total = 1;
            for (int d = 0; d < ndim; ++d) {
                if (shape[d] != 1) {
                    if ((mask >> d) & 1u) { gg.red_size[gg.nred] = shape[d]; gg.red_stride[gg.nred] = stride; ++gg.nred; gg.nred_total *= shape[d]; }
                    else { gg.keep_size[gg.nkeep] = shape[d]; gg.keep_stride[gg.nkeep] = stride; ++gg.nkeep; gg.nout *= shape[d]; }
                }
                stride *= shape[d];
            }
            const bool narrow = gg.nred_total < (1ll << 31);        // element indices fit 32 bits (with the group's stride added)
#define RK_GENERIC(GROUP, BLOCKS)                                                                                            \
    do {                                                                                                                     \
        const int64_t blocks = (BLOCKS);                                                                                     \
        if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;                                                                    \
        if (narrow) reduce_generic_kernel<In, Acc, Xf, Op, Sink, 256, GROUP, uint32_t><<<(unsigned)blocks, 256, 0, stream>>>(A, gg, xf, op, sink); \
        else reduce_generic_kernel<In, Acc, Xf, Op, Sink, 256, GROUP, int64_t><<<(unsigned)blocks, 256, 0, stream>>>(A, gg, xf, op, sink);         \
    } while (0)
            if (gg.nred_total <= 64 && gg.nout >= 16384) RK_GENERIC(1, (gg.nout + 255) / 256);
            else if (gg.nout <= 2048 && gg.nred_total >= 4096) RK_GENERIC(256, gg.nout);
            else RK_GENERIC(64, (gg.nout + 3) / 4);
#undef RK_GENERIC
            break;
        }
    }
    RK_LAUNCH_CHECK();
    return RK_SUCCESS;
}

// ---- typed entry points instantiated once per (in, out) pair ---------------------------------------
struct MapreduceArgs {
    int f, op;                   // f: rk_map, or RK_MAP_PROGRAM with `prog`
    const rk_map_program* prog;
    const void* A; int ndim; const int64_t* shape; uint32_t mask;
    void* R; const void* init;
    void* ws; size_t ws_bytes; hipStream_t stream;
    size_t partials_cap = WS_PARTIALS_BYTES;   // bytes of the partials area this call may use (the caller keeps the rest)
};
struct FindArgs {
    int want_max;
    const void* A; int ndim; const int64_t* shape; uint32_t mask;
    void* vals; int64_t* cart;
    void* ws; size_t ws_bytes; hipStream_t stream;
    const int* slot = nullptr;   // CartesianIndex component per dim of `shape` (nullptr: the dim itself)
};

// Reduced dims that are not neighbours (dims=(1,3); the (1,2,4) of a batch norm): the generic kernel walks every
// output's elements with a stride pattern and reaches a tenth of the bandwidth.  Since op is associative and
// commutative, the lowest run of reduced dims is folded first -- a plain single-run reduction of all the data into
// a temporary at the top of the partials area -- and the remaining dims are reduced from that much smaller array.
// (at most half of the partials area the call may use)

template <typename In, typename Acc, typename Xf, typename Op, typename Out = Acc>
inline int32_t mapreduce_one(const MapreduceArgs& a, const Xf& xf) {
    ReduceSink<Acc, Op, Out> sink{(Out*)a.R, a.init ? (Acc)*(const Out*)a.init : Op::template identity<Acc>(), a.init ? 1 : 0};
    const Shape3 s = collapse3(a.ndim, a.shape, a.mask);
    if (!s.single_run && s.total > 0) {
        // the runs of reduced dims (extents of 1 do not break a run), lowest first
        uint32_t run_mask[RK_MAX_DIMS];
        int64_t run_ext[RK_MAX_DIMS];
        int nruns = 0;
        bool in_run = false;
        for (int d = 0; d < a.ndim; ++d) {
            if (a.shape[d] == 1) continue;
            if ((a.mask >> d) & 1u) {
                if (!in_run) { run_mask[nruns] = 0; run_ext[nruns] = 1; ++nruns; in_run = true; }
                run_mask[nruns - 1] |= 1u << d;
                run_ext[nruns - 1] *= a.shape[d];
            } else in_run = false;
        }
        // Fold one run first into a temporary of total / extent elements: the lowest run if that fits (the
        // rest is then reduced from a compact array), else the longest one (sum of 2 x 3 x 2097152 over dims (1, 3):
        // folding dim 1 leaves 25 MB, folding dim 3 leaves six numbers -- the generic kernel, one thread per output,
        // took 41 ms there).
        int longest = 0;
        for (int r = 1; r < nruns; ++r)
            if (run_ext[r] > run_ext[longest]) longest = r;
        const int candidates[2] = {0, longest};
        Workspace w{};
        if (nruns > 0 && carve_workspace(a.ws, a.ws_bytes, 0, &w)) {
            for (int c = 0; c < 2; ++c) {
                const int r = candidates[c];
                const size_t temp_bytes = ((size_t)(s.total / run_ext[r]) * sizeof(Acc) + 255) & ~(size_t)255;
                if (temp_bytes > a.partials_cap / 2) continue;
                int64_t shape1[RK_MAX_DIMS];
                for (int d = 0; d < a.ndim; ++d) shape1[d] = ((run_mask[r] >> d) & 1u) ? 1 : a.shape[d];
                Acc* temp = (Acc*)((char*)w.partials + a.partials_cap - temp_bytes);
                const size_t cap = a.partials_cap - temp_bytes;
                ReduceSink<Acc, Op> to_temp{temp, Op::template identity<Acc>(), 0};
                const int32_t st = launch_reduce<In, Acc>((const In*)a.A, a.ndim, a.shape, run_mask[r], xf, Op(), to_temp,
                                                          a.ws, a.ws_bytes, a.stream, cap);
                if (st != RK_SUCCESS) return st;
                return launch_reduce<Acc, Acc>((const Acc*)temp, a.ndim, shape1, a.mask & ~run_mask[r], MapXform<Acc, Acc, MapIdentity>(),
                                               Op(), sink, a.ws, a.ws_bytes, a.stream, cap);
            }
        }
    }
    // A long reduced dim behind a short contiguous one (sum(A; dims=2) of a 64 x 1_000_000 array): lanes along `inner` fill
    // a quarter of the strided kernel's 256-column strip (2.8 TB/s), and the narrow kernel moves 4 bytes a lane (32 x N:
    // 3.8 TB/s; with 3 columns it holds 5 TB/s and stays: 3 x 2^24 44.7 against 45.0 us in two launches).  With one or two strips in all (256 x 250_000), the last workgroup of a strip folds hundreds of rows of
    // partials alone.  f consecutive rows are one row of f * inner elements -- the same memory -- so the array is
    // reduced as (f * inner) x (mid / f), with full strips and at least 16 of them where a factor allows, into a
    // temporary, whose f groups of `inner` columns a second, tiny reduction folds.
    // Rows that are no whole number of 16-byte vectors (sum(A; dims=2) of a 4097 x 16000 array) are read 4 bytes a lane,
    // 3 TB/s; four of them together are whole vectors again: 88 -> 47 us.
    if (s.single_run && s.inner >= 4 && s.mid >= 1024 && is_aligned(a.A, 16)) {
        constexpr int64_t VEC = 16 / (int64_t)sizeof(In), COLS = WAVE * VEC;
        constexpr int64_t WANT_TILES = 16;
        const int64_t cols0 = (sizeof(In) >= 4 || s.inner % VEC == 0) ? COLS : WAVE;      // the strided kernel's strip (plan_reduce)
        const int64_t strips0 = (s.inner + cols0 - 1) / cols0;
        const bool poor = cols0 == WAVE || (s.mid >= 4096 && (s.inner < WAVE || s.inner * 10 < strips0 * cols0 * 7 || strips0 * s.outer < 4));
        Workspace w{};
        if (poor && carve_workspace(a.ws, a.ws_bytes, 0, &w)) {
            int64_t pick = 0;
            for (int64_t f = 2; f <= 256 && f * 256 <= s.mid; ++f) {
                const int64_t wide = s.inner * f, strips = (wide + COLS - 1) / COLS;
                if (s.mid % f != 0 || wide % VEC != 0 || wide * 10 < strips * COLS * 9) continue;
                if ((size_t)(wide * s.outer) * sizeof(Acc) + 256 > a.partials_cap / 4) break;
                pick = f;
                if (strips * s.outer >= WANT_TILES) break;
            }
            if (pick > 0) {
                const int64_t f = pick, wide = s.inner * f;
                const size_t temp_bytes = ((size_t)(wide * s.outer) * sizeof(Acc) + 255) & ~(size_t)255;
                Acc* temp = (Acc*)((char*)w.partials + a.partials_cap - temp_bytes);
                const size_t cap = a.partials_cap - temp_bytes;
                const int64_t shape1[3] = {wide, s.mid / f, s.outer}, shape2[3] = {s.inner, f, s.outer};
                ReduceSink<Acc, Op> to_temp{temp, Op::template identity<Acc>(), 0};
                const int32_t st = launch_reduce<In, Acc>((const In*)a.A, 3, shape1, 2u, xf, Op(), to_temp, a.ws, a.ws_bytes, a.stream, cap);
                if (st != RK_SUCCESS) return st;
                return launch_reduce<Acc, Acc>((const Acc*)temp, 3, shape2, 2u, MapXform<Acc, Acc, MapIdentity>(), Op(), sink,
                                               a.ws, a.ws_bytes, a.stream, cap);
            }
        }
    }
    return launch_reduce<In, Acc>((const In*)a.A, a.ndim, a.shape, a.mask, xf, Op(), sink, a.ws, a.ws_bytes, a.stream, a.partials_cap);
}

template <typename In, typename Acc, typename Map, typename Out = Acc>
inline int32_t mapreduce_op(const MapreduceArgs& a) {
    const MapXform<In, Acc, Map> xf;
    switch (a.op) {
        case RK_OP_ADD: return mapreduce_one<In, Acc, MapXform<In, Acc, Map>, OpAdd, Out>(a, xf);
        case RK_OP_MUL: return mapreduce_one<In, Acc, MapXform<In, Acc, Map>, OpMul, Out>(a, xf);
        case RK_OP_MAX: return mapreduce_one<In, Acc, MapXform<In, Acc, Map>, OpMax, Out>(a, xf);
        case RK_OP_MIN: return mapreduce_one<In, Acc, MapXform<In, Acc, Map>, OpMin, Out>(a, xf);
        default: return RK_ERR_INVALID_ARGUMENT;
    }
}

// f as a program (validated by the caller: at most RK_MAP_MAX_TOKENS tokens, stack depth within the registers)
template <typename In, typename Acc>
inline ProgXform<In, Acc> make_prog_xform(const rk_map_program& p) {
    ProgXform<In, Acc> xf{};
    for (int i = 0; i < p.n_tokens; ++i) {
        const uint64_t t = (uint64_t)(p.tokens[i] & 0xff) << ((i & 7) * 8);
        if (i < 8) xf.tokens.lo |= t; else xf.tokens.hi |= t;
    }
    xf.n_tokens = p.n_tokens;
    typedef typename ProgXform<In, Acc>::CT CT;
    for (int k = 0; k < RK_MAP_MAX_CONSTS; ++k)
        xf.c[k] = k < p.n_consts ? (std::is_floating_point<CT>::value ? (CT)p.const_f[k] : (CT)p.const_i[k]) : CT(0);
    return xf;
}
// The three-token programs `x c op` / `c x op` with op one of + - * as x * m + a (AffineXform).
template <typename In, typename Acc>
inline bool affine_of(const rk_map_program& p, AffineXform<In, Acc>* out) {
    typedef typename AffineXform<In, Acc>::CT CT;
    if (p.n_tokens != 3 || p.n_consts < 1) return false;
    const int t0 = p.tokens[0], t1 = p.tokens[1], op = p.tokens[2];
    const bool x_first = t0 == 0 && t1 == 1, c_first = t0 == 1 && t1 == 0;
    if (!x_first && !c_first) return false;
    const CT c = std::is_floating_point<CT>::value ? (CT)p.const_f[0] : (CT)p.const_i[0];
    const CT zero = std::is_floating_point<CT>::value ? (CT)-0.0 : CT(0);
    switch (op) {
        case RK_BC_ADD: *out = {CT(1), c}; return true;
        case RK_BC_SUB:
            if (x_first) *out = {CT(1), std::is_integral<CT>::value ? wrap_mul(c, (CT)-1) : (CT)-c};
            else *out = {(CT)-1, c};
            return true;
        case RK_BC_MUL: *out = {c, zero}; return true;
        default: return false;
    }
}
template <typename In, typename Acc, bool ADD_ONLY = false>
inline int32_t mapreduce_prog(const MapreduceArgs& a) {
    typedef ProgXform<In, Acc> Xf;
    if (a.op == RK_OP_ADD) {
        AffineXform<In, Acc> ax{};
        if (affine_of<In, Acc>(*a.prog, &ax)) return mapreduce_one<In, Acc, AffineXform<In, Acc>, OpAdd>(a, ax);
    }
    const Xf xf = make_prog_xform<In, Acc>(*a.prog);
    if constexpr (ADD_ONLY) return a.op == RK_OP_ADD ? mapreduce_one<In, Acc, Xf, OpAdd>(a, xf) : (int32_t)RK_ERR_UNSUPPORTED;
    else switch (a.op) {
        case RK_OP_ADD: return mapreduce_one<In, Acc, Xf, OpAdd>(a, xf);
        case RK_OP_MUL: return mapreduce_one<In, Acc, Xf, OpMul>(a, xf);
        case RK_OP_MAX: return mapreduce_one<In, Acc, Xf, OpMax>(a, xf);
        case RK_OP_MIN: return mapreduce_one<In, Acc, Xf, OpMin>(a, xf);
        default: return RK_ERR_INVALID_ARGUMENT;
    }
}

template <typename In, typename Acc, typename Out = Acc>
inline int32_t mapreduce_typed(const MapreduceArgs& a) {
    switch (a.f) {
        case RK_MAP_IDENTITY: return mapreduce_op<In, Acc, MapIdentity, Out>(a);
        case RK_MAP_ABS2:     return mapreduce_op<In, Acc, MapAbs2, Out>(a);
        case RK_MAP_ABS:      return mapreduce_op<In, Acc, MapAbs, Out>(a);
        default: return RK_ERR_INVALID_ARGUMENT;
    }
}

template <typename T, typename P>
inline int32_t findminmax_pos(const FindArgs& a, const Shape3& s) {
    ArgSink<T, P> sink{};
    sink.A = (const T*)a.A;
    sink.vals = (T*)a.vals;
    sink.cart = a.cart;
    sink.ndim = a.ndim;
    for (int d = 0; d < a.ndim; ++d) sink.shape[d] = a.shape[d];
    for (int d = 0; d < RK_MAX_DIMS; ++d) sink.slot[d] = (int8_t)(a.slot != nullptr && d < a.ndim ? a.slot[d] : d);
    sink.want_max = a.want_max != 0;
    sink.absolute = !s.single_run;
    sink.g = LineGeom{s.inner, s.mid, s.inner * s.outer};
    if (a.want_max)
        return launch_reduce<T, ArgAcc<T, P>>((const T*)a.A, a.ndim, a.shape, a.mask, ArgXform<T, P, true>(), OpArgKey(), sink, a.ws,
                                              a.ws_bytes, a.stream);
    return launch_reduce<T, ArgAcc<T, P>>((const T*)a.A, a.ndim, a.shape, a.mask, ArgXform<T, P, false>(), OpArgKey(), sink, a.ws,
                                          a.ws_bytes, a.stream);
}

template <typename T>
inline int32_t findminmax_typed(const FindArgs& a) {
    const Shape3 s = collapse3(a.ndim, a.shape, a.mask);
    // 32-bit positions along the line whenever they fit (key + position = one 64-bit word)
    if (s.single_run && s.mid < ((int64_t)1 << 31)) return findminmax_pos<T, int32_t>(a, s);
    return findminmax_pos<T, int64_t>(a, s);
}

// one translation unit per type pair (keeps compile times parallel)
int32_t mapreduce_prog_f32(const MapreduceArgs&);
int32_t mapreduce_prog_f32_i64(const MapreduceArgs&);      // count(pred, A): + only
int32_t mapreduce_prog_f64(const MapreduceArgs&);
int32_t mapreduce_prog_f64_i64(const MapreduceArgs&);
int32_t mapreduce_prog_i32(const MapreduceArgs&);
int32_t mapreduce_prog_i64(const MapreduceArgs&);
int32_t mapreduce_prog_i32_i64(const MapreduceArgs&);
int32_t mapreduce_prog_u8_i64(const MapreduceArgs&);
int32_t mapreduce_f32(const MapreduceArgs&);
int32_t mapreduce_f16(const MapreduceArgs&);
int32_t findminmax_f16(const FindArgs&);
int32_t mapreduce_f64(const MapreduceArgs&);
int32_t mapreduce_i32(const MapreduceArgs&);
int32_t mapreduce_i64(const MapreduceArgs&);
int32_t mapreduce_i32_i64(const MapreduceArgs&);
int32_t mapreduce_u8_i64(const MapreduceArgs&);
int32_t mapreduce_u8(const MapreduceArgs&);
int32_t mapreduce_u32(const MapreduceArgs&);
int32_t mapreduce_u32_u64(const MapreduceArgs&);
int32_t mapreduce_u64(const MapreduceArgs&);
int32_t findminmax_u32(const FindArgs&);
int32_t findminmax_u64(const FindArgs&);
int32_t findminmax_u8(const FindArgs&);
int32_t mapreduce_i8_i64(const MapreduceArgs&);
int32_t mapreduce_i8(const MapreduceArgs&);
int32_t findminmax_i8(const FindArgs&);
int32_t mapreduce_i16_i64(const MapreduceArgs&);
int32_t mapreduce_i16(const MapreduceArgs&);
int32_t findminmax_i16(const FindArgs&);
int32_t mapreduce_u16_u64(const MapreduceArgs&);
int32_t mapreduce_u16(const MapreduceArgs&);
int32_t findminmax_u16(const FindArgs&);
int32_t findminmax_f32(const FindArgs&);
int32_t findminmax_f64(const FindArgs&);
int32_t findminmax_i32(const FindArgs&);
int32_t findminmax_i64(const FindArgs&);

}  // namespace rk
