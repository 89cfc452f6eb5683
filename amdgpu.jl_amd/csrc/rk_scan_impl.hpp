// Scan kernels: accumulate / cumsum / cumprod along one dimension of a column-major array.
// Replaces the AcceleratedKernels kernels that src/kernels/accumulate.jl:1-8 forwards to.
//
// The array is seen as (inner, mid, outer) with `mid` scanned.
//   inner == 1 : contiguous lines of length mid
//       scan_lookback_kernel   single pass, decoupled look-back (Merrill & Garland): every
//                              workgroup scans one tile of a line in registers, publishes the
//                              tile aggregate, resolves its exclusive prefix by looking back
//                              over the predecessors' descriptors, and writes once.  8 B/elt.
//       scan_wave_lines_kernel lines shorter than a tile: one wave per line with a running carry
//   inner  > 1 : strided lines, lanes run along the contiguous `inner` axis
//       scan_strided_kernel    4 waves x register tiles of rows, column totals through LDS
//       scan_rows_ordered_kernel  few strips of columns, many rows: tiles of rows in launch order, single pass
//       scan_rows_packed_kernel   rows of 128 bytes up to half a strip: several rows per load instruction, single pass
//       scan_cols_kernel       a scanned extent <= 16 behind >= 64 contiguous columns: a lane per group of columns
//       scan_narrow_kernel     1 < inner < 64 with long lines: tiles of whole rows through LDS
//   scan_thread_kernel         one lane per line (tiny lines)
//   scan_lds_lines_kernel      short lines of any length (contiguous, or short along a narrow inner): whole slabs through LDS
#pragma once

#include "rk_common.hpp"

namespace rk {

// ---- tile descriptors of the look-back scan ---------------------------------------------------
// One 64-bit word per 32-bit slice of the value: low half = payload, high half = tag
// (epoch << 2 | status).  A word is stored / loaded with one relaxed agent-scope atomic, so the
// payload always travels with its tag and no fence is needed.  A value of several words is valid
// when all its tags agree.  Descriptors whose epoch differs from the current call's are stale.
constexpr uint32_t DESC_A = 1;   // tile aggregate available
constexpr uint32_t DESC_P = 2;   // inclusive prefix available

template <typename T>
__device__ __forceinline__ void desc_publish(uint64_t* desc, int64_t stride, int64_t tile, T value, uint32_t tag) {
    Words<T> w = to_words(value);
#pragma unroll
    for (int i = 0; i < Words<T>::N; ++i)
        __hip_atomic_store(&desc[i * stride + tile], ((uint64_t)tag << 32) | (uint64_t)w.w[i], __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
}

// Reads one descriptor value; returns its status (0 = not of this call / not yet written).
template <typename T>
__device__ __forceinline__ uint32_t desc_read(const uint64_t* desc, int64_t stride, int64_t idx, uint32_t tagA, uint32_t tagP,
                                              Words<T>& val) {
    uint32_t status = 0;
#pragma unroll
    for (int i = 0; i < Words<T>::N; ++i) {
        const uint64_t d = __hip_atomic_load(&desc[i * stride + idx], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t tag = (uint32_t)(d >> 32);
        val.w[i] = (uint32_t)d;
        const uint32_t st = tag == tagA ? DESC_A : (tag == tagP ? DESC_P : 0u);
        status = (i == 0) ? st : (st == status ? st : 0u);
    }
    return status;
}

// Two-level decoupled look-back; executed by one full wave, returns the wave-uniform exclusive
// prefix of `tile` inside its line.
//
// With one level, a tile can only finish once it sees an *inclusive* prefix within the 64
// descriptors it polls at a time, so inclusive prefixes advance at most 64 tiles per poll round trip
// (a device-coherent load: microseconds under load) -- far below the tile rate 8 TB/s needs.  Here
// the tiles of a line form groups of 64.  A tile sums the plain aggregates of the predecessors inside
// its group (they depend on nobody, so they appear as soon as those tiles have read their data), and
// takes the rest from group descriptors: the last tile of a group publishes the group aggregate (GA)
// as soon as its in-group sum is complete and the inclusive prefix at the group end (GP) when it has
// its own prefix.  One poll of 64 group descriptors spans 4096 tiles, so the two polls (issued
// together) normally resolve in one or two round trips whatever the distance to the nearest
// inclusive prefix.
//   tl   index of the tile in its line          gl   global index of the tile's group
//   agg  aggregate of this tile (already published by the caller as the tile's descriptor)
template <typename T, typename Op>
__device__ __forceinline__ T desc_lookback2(uint64_t* tile_desc, int64_t tstride, uint64_t* group_desc, int64_t gstride,
                                            int64_t tile, int64_t tl, int64_t gl, uint32_t epoch, T agg, T init, Op op, T ident,
                                            const WaitCtl& wc) {
    const int lane = lane_id();
    const uint32_t tagA = (epoch << 2) | DESC_A, tagP = (epoch << 2) | DESC_P;
    const int r = (int)(tl & (WAVE - 1));           // predecessors inside the group
    const int64_t g = tl >> 6;                      // groups in front of this one in the line
    const int64_t t0 = tile - r;
    T local = ident, gacc = ident, gpre = init;
    bool local_done = (r == 0), group_done = (g == 0), ga_published = false;
    int64_t gfirst = gl - 1, grem = g;              // nearest group of the current window, groups left
    long long rounds = 0;
    while (!(local_done && group_done)) {
        Words<T> tv = to_words(ident), gv = to_words(ident);
        uint32_t tstat = DESC_A, gstat = DESC_P;    // lanes outside the range: terminators holding ident
        if (!local_done && lane < r) tstat = desc_read<T>(tile_desc, tstride, t0 + lane, tagA, tagP, tv);
        if (!group_done && lane < grem) gstat = desc_read<T>(group_desc, gstride, gfirst - lane, tagA, tagP, gv);
        if (!local_done && __ballot(tstat == 0u) == 0ull) {
            local = wave_reduce(from_words<T>(tv), op);
            local_done = true;
        }
        if (local_done && r == WAVE - 1 && !ga_published && !group_done) {
            if (lane == 0) desc_publish(group_desc, gstride, gl, op(local, agg), tagA);
            ga_published = true;
        }
        if (!group_done) {
            const uint64_t ballotP = __ballot(gstat == DESC_P);
            const uint64_t ballotX = __ballot(gstat == 0u);
            const int np = ballotP ? (__ffsll((unsigned long long)ballotP) - 1) : -1;
            const uint64_t needed = np >= 0 ? ((1ull << np) - 1ull) : ~0ull;
            if ((ballotX & needed) == 0ull) {
                const T x = (np < 0 || lane <= np) ? from_words<T>(gv) : ident;
                gacc = op(wave_reduce(x, op), gacc);
                if (np >= 0) {
                    group_done = true;
                    // a real GP already contains init; running off the line start does not
                    gpre = (np >= grem) ? op(init, gacc) : gacc;
                } else {
                    gfirst -= WAVE;
                    grem -= WAVE;
                }
            }
        }
        if (!(local_done && group_done) && wait_give_up(wc, rounds)) break;     // the prefix below is then meaningless
    }
    const T prefix = op(gpre, local);
    if (r == WAVE - 1 && lane == 0) desc_publish(group_desc, gstride, gl, op(prefix, agg), tagP);
    return prefix;
}

// ---- look-back with group leaders ------------------------------------------------------------------------------
// In desc_lookback2 every waiting tile polls the descriptors of the nearest groups, so the one or two 128-byte lines
// that hold them are read by every tile in flight, round after round.  Device-coherent accesses to one line are
// served one at a time (some 10 ns each on MI355X): with thousands of tiles in flight that line, not HBM, sets the
// pace -- measured as 7 ns per tile whatever the tile size, occupancy or polling discipline.  Here only the FIRST
// tile of a group of 64 (its leader) looks at the group level: it sums group aggregates back to the nearest inclusive
// prefix and publishes the result -- the inclusive prefix through the previous group -- into that group's descriptor;
// the other 63 tiles sum the aggregates of their predecessors inside the group and wait for that one word.  Every
// group descriptor has a 128-byte line of its own (word i of group g at g * GROUP_DESC_STRIDE + i), so its readers are
// the 63 tiles of the next group and the few leaders in flight.  Per tile the cost falls to ~1.5 ns.
//   tile descriptors   [words][ntiles], DESC_A only           group descriptors   DESC_A: aggregate of the group
//                                                                                 DESC_P: inclusive prefix through it
constexpr int GROUP_DESC_STRIDE = 16;      // 64-bit words: one 128-byte line per group

template <typename T>
__device__ __forceinline__ void gdesc_publish(uint64_t* gd, int64_t g, T value, uint32_t tag) {
    Words<T> w = to_words(value);
    static_assert(Words<T>::N <= GROUP_DESC_STRIDE, "a value fits the line of its group");
#pragma unroll
    for (int i = 0; i < Words<T>::N; ++i)
        __hip_atomic_store(&gd[g * GROUP_DESC_STRIDE + i], ((uint64_t)tag << 32) | (uint64_t)w.w[i], __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T>
__device__ __forceinline__ uint32_t gdesc_read(const uint64_t* gd, int64_t g, uint32_t tagA, uint32_t tagP, Words<T>& val) {
    uint32_t status = 0;
#pragma unroll
    for (int i = 0; i < Words<T>::N; ++i) {
        const uint64_t d = __hip_atomic_load(&gd[g * GROUP_DESC_STRIDE + i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t tag = (uint32_t)(d >> 32);
        val.w[i] = (uint32_t)d;
        const uint32_t st = tag == tagA ? DESC_A : (tag == tagP ? DESC_P : 0u);
        status = (i == 0) ? st : (st == status ? st : 0u);
    }
    return status;
}

// Forward progress.  A tile that waits depends on workgroups that must be running.  With tile numbers taken from the
// launch order that holds for one grid alone on the device (workgroups start in index order), but two such grids
// resident together can in principle starve each other of slots: the lowest unfinished tile of each waiting for a slot
// that waiting tiles of the other hold.  So no wait here is open-ended: after `wait_patience` unsuccessful polls the
// tile stops waiting and resolves its prefix ALONE (desc_lookback_alone): whatever a predecessor has not published it
// computes itself from the input -- `agg_of(p)` returns the aggregate of tile p of the same line, computed by the
// calling wave -- and publishes in the predecessor's name, so nobody else has to repeat it.  Such a tile needs no other
// workgroup at all; the call's result is the same (bit for bit for integers; float sums may associate differently, as
// they do between any two runs).  `helped` counts the tiles that took this path (WsHeader::alone), for tests and
// curiosity.  The wait budget proper (RK_ERR_WAIT) is left to kernels that cannot help themselves.
constexpr long long WAIT_PATIENCE = 4096;       // polls (a microsecond or two each) before a tile helps itself

struct WaitAlone {
    long long patience;      // min(WAIT_PATIENCE, the wait budget): tests set a budget of 1 to send every tile this way
    uint32_t* counter;       // WsHeader::alone
};
__device__ __forceinline__ bool wait_expired(const WaitAlone& w, const WaitCtl& wc, long long& rounds) {
    if (++rounds >= w.patience) return true;
    for (int b = 0; b < wc.backoff; ++b) __builtin_amdgcn_s_sleep(8);
    return false;
}

// Sum of the aggregates of tiles first .. first + count - 1 (count <= 64) without waiting: missing ones are computed
// from the input and published.  One full wave; the result is wave-uniform.
template <typename T, typename Op, typename Agg>
__device__ __forceinline__ T desc_sum_or_compute(uint64_t* tile_desc, int64_t tstride, int64_t first, int count, uint32_t tagA, uint32_t tagP,
                                                 Op op, T ident, const Agg& agg_of) {
    const int lane = lane_id();
    Words<T> tv = to_words(ident);
    uint32_t st = DESC_A;
    if (lane < count) st = desc_read<T>(tile_desc, tstride, first + lane, tagA, tagP, tv);
    unsigned long long missing = __ballot(st == 0u);
    T sum = wave_reduce(st == 0u ? ident : from_words<T>(tv), op);
    while (missing != 0ull) {
        const int l = __ffsll(missing) - 1;
        missing &= missing - 1ull;
        T a = agg_of(first + l);
        // In place (out == in) the tile's own workgroup may have started meanwhile and be storing its results over the
        // elements just read.  It publishes its aggregate before it stores anything (publish, look-back, stores; the
        // first tile of a line waits for its publication), so the descriptor is read once more, AFTER the elements: still
        // empty means no store had begun when the reads finished and `a` is sound; published means the owner's value is
        // there to take, whatever was read.
        asm volatile("" : "+v"(a) : : "memory");          // the descriptor's load is issued behind the reads that made `a`
        Words<T> again = to_words(ident);
        uint32_t st2 = 0;
        if (lane == 0) st2 = desc_read<T>(tile_desc, tstride, first + l, tagA, tagP, again);
        st2 = (uint32_t)__builtin_amdgcn_readfirstlane((int)st2);
        if (st2 != 0u) a = read_lane(from_words<T>(again), 0);
        else if (lane == 0) desc_publish(tile_desc, tstride, first + l, a, tagA);
        sum = op(sum, a);
    }
    return sum;
}

// The exclusive prefix of `tile` with no help from anybody (see above).  One full wave.
template <typename T, typename Op, typename Agg>
__device__ __forceinline__ T desc_lookback_alone(uint64_t* tile_desc, int64_t tstride, uint64_t* gd, int64_t tile, int64_t tl, int64_t gl,
                                              uint32_t epoch, T agg, T init, Op op, T ident, const Agg& agg_of, uint32_t* alone_counter) {
    const int lane = lane_id();
    const uint32_t tagA = (epoch << 2) | DESC_A, tagP = (epoch << 2) | DESC_P;
    const int r = (int)(tl & (WAVE - 1));
    const int64_t g = tl >> 6;
    const int64_t t0 = tile - r;
    if (lane == 0) __hip_atomic_fetch_add(alone_counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    auto group_status = [&](int64_t k, T& value) -> uint32_t {
        Words<T> gv = to_words(ident);
        uint32_t st = 0;
        if (lane == 0) st = gdesc_read<T>(gd, k, tagA, tagP, gv);
        value = read_lane(from_words<T>(gv), 0);
        return (uint32_t)__builtin_amdgcn_readfirstlane((int)st);
    };
    const T local = r > 0 ? desc_sum_or_compute(tile_desc, tstride, t0, r, tagA, tagP, op, ident, agg_of) : ident;
    if (r == WAVE - 1) {                          // the group's aggregate, unless the descriptor already says as much or more
        T seen;
        if (group_status(gl, seen) == 0u && lane == 0) gdesc_publish(gd, gl, op(local, agg), tagA);
    }
    T base = init;
    if (g > 0) {
        T acc = ident;
        bool found = false;
        for (int64_t k = gl - 1; k >= gl - g; --k) {          // the groups of this line in front, nearest first
            T x;
            const uint32_t st = group_status(k, x);
            if (st == DESC_P) {
                base = op(x, acc);                             // a published prefix contains init
                found = true;
                break;
            }
            if (st == 0u) {
                x = desc_sum_or_compute(tile_desc, tstride, t0 - (gl - k) * WAVE, WAVE, tagA, tagP, op, ident, agg_of);
                T seen;
                if (group_status(k, seen) == 0u && lane == 0) gdesc_publish(gd, k, x, tagA);
            }
            acc = op(x, acc);
        }
        if (!found) base = op(init, acc);
        if (lane == 0) gdesc_publish(gd, gl - 1, base, tagP);  // what the group's leader publishes, for the other tiles of the group
    }
    return op(base, local);
}

// Executed by one full wave; returns the wave-uniform exclusive prefix of `tile` (tl > 0) inside its line.
//   tl  index of the tile in its line     gl  global index of the tile's group     agg  aggregate of this tile
// `expired`: the patience ran out; the value returned is then meaningless and the caller resolves the prefix with
// desc_lookback_alone (one call site, where it can first put registers it holds aside).
template <typename T, typename Op>
__device__ __forceinline__ T desc_lookback_leader(uint64_t* tile_desc, int64_t tstride, uint64_t* gd, int64_t tile, int64_t tl, int64_t gl,
                                                  uint32_t epoch, T agg, T init, Op op, T ident, const WaitCtl& wc, const WaitAlone& wa,
                                                  bool& expired) {
    const int lane = lane_id();
    const uint32_t tagA = (epoch << 2) | DESC_A, tagP = (epoch << 2) | DESC_P;
    const int r = (int)(tl & (WAVE - 1));           // predecessors inside the group
    const int64_t g = tl >> 6;                      // groups in front of this one in the line
    long long rounds = 0;
    if (r == 0) {
        // leader (g > 0, since tl > 0): aggregates of the groups in front, back to the nearest inclusive prefix
        T gacc = ident, base = init;
        int64_t gfirst = gl - 1, grem = g;
        for (;;) {
            Words<T> gv = to_words(ident);
            uint32_t gstat = DESC_P;                // lanes beyond the line start: terminators holding ident
            if (lane < grem) gstat = gdesc_read<T>(gd, gfirst - lane, tagA, tagP, gv);
            const uint64_t ballotP = __ballot(gstat == DESC_P);
            const uint64_t ballotX = __ballot(gstat == 0u);
            const int np = ballotP ? (__ffsll((unsigned long long)ballotP) - 1) : -1;
            const uint64_t needed = np >= 0 ? ((1ull << np) - 1ull) : ~0ull;
            if ((ballotX & needed) == 0ull) {
                const T x = (np < 0 || lane <= np) ? from_words<T>(gv) : ident;
                gacc = op(wave_reduce(x, op), gacc);
                if (np >= 0) {
                    base = (np >= grem) ? op(init, gacc) : gacc;     // a real prefix already contains init
                    break;
                }
                gfirst -= WAVE;
                grem -= WAVE;
                continue;
            }
            if (wait_expired(wa, wc, rounds)) { expired = true; return ident; }
        }
        if (lane == 0) gdesc_publish(gd, gl - 1, base, tagP);
        return base;
    }
    const int64_t t0 = tile - r;
    T local = ident;
    for (;;) {
        Words<T> tv = to_words(ident);
        uint32_t tstat = DESC_A;
        if (lane < r) tstat = desc_read<T>(tile_desc, tstride, t0 + lane, tagA, tagP, tv);
        if (__ballot(tstat == 0u) == 0ull) {
            local = wave_reduce(from_words<T>(tv), op);
            break;
        }
        if (wait_expired(wa, wc, rounds)) { expired = true; return ident; }
    }
    if (r == WAVE - 1 && lane == 0) gdesc_publish(gd, gl, op(local, agg), tagA);
    T base = init;
    if (g > 0) {
        for (;;) {
            Words<T> gv = to_words(ident);
            uint32_t st = 0;
            if (lane == 0) st = gdesc_read<T>(gd, gl - 1, tagA, tagP, gv);
            st = (uint32_t)__builtin_amdgcn_readfirstlane((int)st);
            if (st == DESC_P) {
                base = read_lane(from_words<T>(gv), 0);
                break;
            }
            if (wait_expired(wa, wc, rounds)) { expired = true; return ident; }
        }
    }
    return op(base, local);
}

struct ScanGeom {
    int64_t inner, mid, outer;
};

// ---- one tile of a contiguous line, scanned in registers ---------------------------------------------
// NW waves x K loads of 16 output bytes.  Wave w owns the w-th part of the tile; its k-th load covers 64 * VEC
// consecutive elements (one fully coalesced 1 KiB request for 4-byte inputs).  Per load: scan inside the lane, DPP scan
// across the wave, carry to the next load; the prefix inside the wave's part is folded into the values at once, so
// a tile costs K vector registers and nothing else (a separate array of per-load prefixes cost K more registers and
// kept the 1024-thread kernel at one workgroup per compute unit).  Exclusive scans shift while folding.
template <typename T, int K> struct TileRegs {
    static constexpr int VEC = 16 / sizeof(T);
    // vector values, not T v[K][VEC]: with the array form the 64-bit integer instantiations kept the tile in private
    // memory (a store and a load per element: cumsum of Int64[2^26] 342 us against 191 us for Float64)
    typename VecOf<T, VEC>::type v[K];     // scan of the wave's part up to and including (inclusive) / excluding the element
};

// Vectors at element-aligned addresses (load_nt_elems) exist for 4- and 8-byte elements; for the rest these are
// never called (value == false) but must compile.
template <typename In, typename T, bool OK = (sizeof(In) >= 4 && sizeof(T) >= 4)> struct ElemVectors {
    static constexpr bool value = true;
    template <int N> static __device__ __forceinline__ typename VecOf<In, N>::type load(const In* p) { return load_nt_elems<In, N>(p); }
    template <int N> static __device__ __forceinline__ void store(In* p, typename VecOf<In, N>::type v) { store_nt_elems<In, N>(p, v); }
};
template <typename In, typename T> struct ElemVectors<In, T, false> {
    static constexpr bool value = false;
    template <int N> static __device__ __forceinline__ typename VecOf<In, N>::type load(const In*) { return typename VecOf<In, N>::type{}; }
    template <int N> static __device__ __forceinline__ void store(In*, typename VecOf<In, N>::type) {}
};

// ---- stores of scan results ---------------------------------------------------------------------------------------------
// The kernels compute in T; the array they fill holds Out: T itself, or a narrower type that is scanned in the next
// wider one -- Int8 / Int16 in Int32, UInt8 / UInt16 in UInt32: the store keeps the low bits, which is the narrow type's
// own wrap-around for + and * and the value itself for max / min; Float16 in Float32, rounded once at the store.
template <typename Out, typename T, int N>
__device__ __forceinline__ void out_store_nt(Out* p, typename VecOf<T, N>::type v) {        // p aligned to N * sizeof(Out)
    if constexpr (std::is_same<Out, T>::value) store_nt((typename VecOf<T, N>::type*)p, v);
    else if constexpr (N == 1) *p = (Out)v;
    else {
        typename VecOf<Out, N>::type o;
#pragma unroll
        for (int j = 0; j < N; ++j) o[j] = (Out)v[j];
        store_nt((typename VecOf<Out, N>::type*)p, o);
    }
}
// A vector at an element-aligned address: only where the stored type is the computed one, of 4 or 8 bytes.
template <typename Out, typename T> struct OutElemVectors { static constexpr bool value = std::is_same<Out, T>::value && sizeof(T) >= 4; };
template <typename Out, typename T, int N>
__device__ __forceinline__ void out_store_elems(Out* p, typename VecOf<T, N>::type v) {
    if constexpr (OutElemVectors<Out, T>::value) store_nt_elems<T, N>(p, v);
}

// The values of a wave's part, loaded into r, scanned in place; returns the total of the part.
template <typename T, typename Op, int K>
__device__ __forceinline__ T tile_scan_regs(int inclusive, Op op, TileRegs<T, K>& r) {
    constexpr int VEC = 16 / sizeof(T);
    const T ident = Op::template identity<T>();
    T carry = ident;
#pragma unroll
    for (int k = 0; k < K; ++k) {
#pragma unroll
        for (int j = 1; j < VEC; ++j) r.v[k][j] = op(r.v[k][j - 1], r.v[k][j]);
        const T inc = wave_scan_inclusive(r.v[k][VEC - 1], op, ident);
        const T excl = op(carry, wave_shift_right(inc, ident));
        carry = op(carry, read_lane(inc, WAVE - 1));
        if (inclusive) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) r.v[k][j] = op(excl, r.v[k][j]);
        } else {
#pragma unroll
            for (int j = VEC - 1; j > 0; --j) r.v[k][j] = op(excl, r.v[k][j - 1]);
            r.v[k][0] = excl;
        }
        // 8-byte values: one vector at a time.  Interleaved, the wave scans of several vectors (two registers a value,
        // no DPP form of the 64-bit operators) need more temporaries than the 64-register kernels have left
        if constexpr (sizeof(T) == 8) asm volatile("" : "+v"(r.v[k]));
    }
    return carry;
}

template <typename In, typename T, typename Op, bool VECTOR, int K, int NW = 4>
__device__ __forceinline__ T tile_load_scan(const In* __restrict__ in, int64_t e0, int valid, int inclusive, Op op, TileRegs<T, K>& r) {
    constexpr int VEC = 16 / sizeof(T);
    constexpr int TILE = NW * WAVE * VEC * K;
    typedef typename VecOf<In, VEC>::type VI;
    const T ident = Op::template identity<T>();
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int woff = wave * (WAVE * VEC * K) + lane * VEC;
    if (VECTOR && valid == TILE) {
        const In* p = in + e0 + woff;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const VI x = load_nt((const VI*)(p + k * WAVE * VEC));
#pragma unroll
            for (int j = 0; j < VEC; ++j) r.v[k][j] = (T)x[j];
        }
    } else if (!VECTOR && ElemVectors<In, T>::value && valid == TILE) {
        // a full tile of a line that starts at an odd address: the same loads at element-aligned addresses
        const In* p = in + e0 + woff;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const VI x = ElemVectors<In, T>::template load<VEC>(p + k * WAVE * VEC);
#pragma unroll
            for (int j = 0; j < VEC; ++j) r.v[k][j] = (T)x[j];
        }
    } else if (VECTOR && valid % VEC == 0) {
        // a tile that its line does not fill (every line of cumsum(A; dims=1) on a 3000 x N array): whole vectors all
        // the same, and every lane issues its K loads unconditionally -- a vector past the end reads the tile's first
        // one and drops it -- because a load under a condition of its own is waited for before the next is issued
        // (element-wise conditional loads: 3000 x 20000 Float32 143 us, 3.4 TB/s, against 6.2 TB/s for 4096 x 16384)
        const In* p = in + e0;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int idx = woff + k * WAVE * VEC;
            const bool have = idx < valid;
            const VI x = load_nt((const VI*)(p + (have ? idx : 0)));
#pragma unroll
            for (int j = 0; j < VEC; ++j) r.v[k][j] = have ? (T)x[j] : ident;
        }
    } else if (ElemVectors<In, T>::value && valid >= VEC) {
        // lines that start at odd addresses, or whose length is no whole number of vectors: global memory takes 16-byte
        // accesses at any element-aligned address, so only the one vector the line's end cuts goes element by element.
        // Unconditional loads again (a vector past the end reads the tile's first).
        const In* p = in + e0;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int idx = woff + k * WAVE * VEC;
            const bool whole = idx + VEC <= valid;
            const VI x = ElemVectors<In, T>::template load<VEC>(p + (whole ? idx : 0));
#pragma unroll
            for (int j = 0; j < VEC; ++j) r.v[k][j] = whole ? (T)x[j] : ident;
            if (!whole && idx < valid) {
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    if (idx + j < valid) r.v[k][j] = (T)p[idx + j];
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const int idx = woff + k * WAVE * VEC + j;
                const bool have = idx < valid;
                const T x = (T)in[e0 + (have ? idx : 0)];
                r.v[k][j] = have ? x : ident;
            }
    }
    return tile_scan_regs<T, Op, K>(inclusive, op, r);
}

// `base`: everything in front of this wave's part (init, earlier tiles, earlier waves).
template <typename Out, typename T, typename Op, bool VECTOR, int K, int NW = 4>
__device__ __forceinline__ void tile_store(Out* __restrict__ out, int64_t e0, int valid, T base, Op op, const TileRegs<T, K>& r) {
    constexpr int VEC = 16 / sizeof(T);
    constexpr int TILE = NW * WAVE * VEC * K;
    typedef typename VecOf<T, VEC>::type VT;
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int woff = wave * (WAVE * VEC * K) + lane * VEC;
    if (VECTOR && valid == TILE) {
        Out* p = out + e0 + woff;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            VT o;
#pragma unroll
            for (int j = 0; j < VEC; ++j) o[j] = op(base, r.v[k][j]);
            out_store_nt<Out, T, VEC>(p + k * WAVE * VEC, o);
        }
    } else if (!VECTOR && OutElemVectors<Out, T>::value && valid == TILE) {
        Out* p = out + e0 + woff;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            VT o;
#pragma unroll
            for (int j = 0; j < VEC; ++j) o[j] = op(base, r.v[k][j]);
            out_store_elems<Out, T, VEC>(p + k * WAVE * VEC, o);
        }
    } else if (VECTOR && valid % VEC == 0) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int idx = woff + k * WAVE * VEC;
            VT o;
#pragma unroll
            for (int j = 0; j < VEC; ++j) o[j] = op(base, r.v[k][j]);
            if (idx < valid) out_store_nt<Out, T, VEC>(out + e0 + idx, o);
        }
    } else if (OutElemVectors<Out, T>::value) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int idx = woff + k * WAVE * VEC;
            VT o;
#pragma unroll
            for (int j = 0; j < VEC; ++j) o[j] = op(base, r.v[k][j]);
            if (idx + VEC <= valid) out_store_elems<Out, T, VEC>(out + e0 + idx, o);
            else if (idx < valid) {
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    if (idx + j < valid) out[e0 + idx + j] = (Out)o[j];
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const int idx = woff + k * WAVE * VEC + j;
                if (idx < valid) out[e0 + idx] = (Out)op(base, r.v[k][j]);
            }
    }
}

// ---- tiles of 1- and 2-byte integers, kept packed ------------------------------------------------------------------------
// A tile of the single-pass scan lives as long whatever it holds (its loads, a look-back, its stores), so what counts is
// the bytes it moves.  Widened to 32-bit registers, 32 registers a lane hold 32 elements: 64 KiB of Int16, 32 KiB of Int8
// a tile.  Here the registers keep the 16-byte vectors as they were loaded -- 8 or 16 elements each -- and a vector is
// unpacked only while it is scanned and again when the tile's prefix is added: 128 KiB of input a tile like the 4-byte
// types.  The values between the two steps are the scan without the tile's prefix, truncated to the element type: for
// + and * that is the type's own wrap-around (the low bits of a sum or product depend on the low bits of the operands
// only), for max / min / & / | / xor the values never leave the type's range.  Lines of whole, 16-byte aligned vectors.
typedef uint32_t PackedVec __attribute__((ext_vector_type(4)));
template <typename In, typename T> struct Packed {
    static_assert(std::is_integral<In>::value && sizeof(In) <= 2 && sizeof(T) == 4, "1- and 2-byte integers in 32-bit registers");
    static constexpr int PV = 16 / (int)sizeof(In);           // elements per vector
    static constexpr int PW = 4 / (int)sizeof(In);            // elements per 32-bit word
    static constexpr int BITS = 8 * (int)sizeof(In);
    static __device__ __forceinline__ void unpack_word(uint32_t w, T (&e)[PW]) {
#pragma unroll
        for (int h = 0; h < PW; ++h) e[h] = (T)(In)(w >> (h * BITS));          // sign- or zero-extends
    }
    static __device__ __forceinline__ uint32_t pack_word(const T (&e)[PW]) {
        typedef typename std::make_unsigned<In>::type UIn;
        uint32_t x = 0;
#pragma unroll
        for (int h = 0; h < PW; ++h) x |= (uint32_t)(UIn)e[h] << (h * BITS);
        return x;
    }
    template <typename Op> static __device__ __forceinline__ T total(const PackedVec& v, Op op) {
        T e[PW];
        unpack_word(v[0], e);
        T t = e[0];
#pragma unroll
        for (int h = 1; h < PW; ++h) t = op(t, e[h]);
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            unpack_word(v[w], e);
#pragma unroll
            for (int h = 0; h < PW; ++h) t = op(t, e[h]);
        }
        return t;
    }
    static __device__ __forceinline__ PackedVec splat(T x) {
        T e[PW];
#pragma unroll
        for (int h = 0; h < PW; ++h) e[h] = x;
        const uint32_t w = pack_word(e);
        return PackedVec{w, w, w, w};
    }
};
template <int K> struct PackedRegs { PackedVec v[K]; };

template <typename In, typename T, typename Op, int K, int NW>
__device__ __forceinline__ T packed_tile_load_scan(const In* __restrict__ in, int64_t e0, int valid, int inclusive, Op op, PackedRegs<K>& r) {
    typedef Packed<In, T> P;
    constexpr int PV = P::PV;
    constexpr int TILE = NW * WAVE * PV * K;
    // the identity of the ELEMENT type: it is packed with the values (exclusive scans store it, short tiles are padded
    // with it), and the 32-bit one of max / min does not survive the truncation
    const T ident = (T)Op::template identity<In>();
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int woff = wave * (WAVE * PV * K) + lane * PV;
    const In* p = in + e0 + woff;
    if (valid == TILE) {
#pragma unroll
        for (int k = 0; k < K; ++k) r.v[k] = load_nt((const PackedVec*)(p + k * WAVE * PV));
    } else {
        // a tile that its line does not fill (valid is a whole number of vectors): every lane still issues its K loads
        // unconditionally -- a vector past the end reads the tile's first one and becomes a vector of identities
        const PackedVec idv = P::splat(ident);
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const bool have = woff + k * WAVE * PV < valid;
            const PackedVec x = load_nt((const PackedVec*)(have ? p + k * WAVE * PV : in + e0));
            r.v[k] = have ? x : idv;
        }
    }
    // Per vector: the lane's total first (elements unpacked on the fly), the scan of the totals across the wave, then
    // word by word a running scan from the lane's exclusive prefix -- four or two elements unpacked at a time.
    T carry = ident;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const T total = P::total(r.v[k], op);
        const T inc = wave_scan_inclusive(total, op, ident);
        T run = op(carry, wave_shift_right(inc, ident));
        carry = op(carry, read_lane(inc, WAVE - 1));
        PackedVec o;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            T e[P::PW], x[P::PW];
            P::unpack_word(r.v[k][w], e);
#pragma unroll
            for (int h = 0; h < P::PW; ++h) {
                const T before = run;
                run = op(run, e[h]);
                x[h] = inclusive ? run : before;
            }
            o[w] = P::pack_word(x);
        }
        r.v[k] = o;
        // packed here and now: left to itself the compiler keeps the unpacked values of several vectors alive and
        // packs them late, which spilled 16 registers
        asm volatile("" : "+v"(r.v[k]));
    }
    return carry;
}

template <typename In, typename T, typename Op, int K, int NW>
__device__ __forceinline__ void packed_tile_store(In* __restrict__ out, int64_t e0, int valid, T base, Op op, const PackedRegs<K>& r) {
    typedef Packed<In, T> P;
    constexpr int PV = P::PV;
    constexpr int TILE = NW * WAVE * PV * K;
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int woff = wave * (WAVE * PV * K) + lane * PV;
    In* p = out + e0 + woff;
    const bool full = valid == TILE;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        PackedVec o;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            T e[P::PW];
            P::unpack_word(r.v[k][w], e);
#pragma unroll
            for (int h = 0; h < P::PW; ++h) e[h] = op(base, e[h]);
            o[w] = P::pack_word(e);
        }
        if (full || woff + k * WAVE * PV < valid) store_nt((PackedVec*)(p + k * WAVE * PV), o);
    }
}

// Aggregate of another tile of the same line, computed from the input by the calling wave (the look-back's way out
// when that tile's workgroup is not there to publish it: desc_lookback_alone).  Lines of whole, aligned vectors; every
// tile in front of another is full.
template <typename In, typename T, typename Op, int TILE, bool VECTOR = true> struct ScanTileAggregate {
    const In* first;        // first element of the asking tile
    int64_t   tile;         // its number
    __device__ __forceinline__ T operator()(int64_t p) const {
        constexpr int VEC = 16 / sizeof(T);
        typedef typename VecOf<In, VEC>::type VI;
        const Op op;
        const In* q = first - (tile - p) * (int64_t)TILE;
        T acc = Op::template identity<T>();
        for (int i = lane_id() * VEC; i < TILE; i += WAVE * VEC) {
            VI x;
            if constexpr (VECTOR) x = *(const VI*)(q + i);
            else x = ElemVectors<In, T>::template load<VEC>(q + i);        // lines at element-aligned addresses
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc = op(acc, (T)x[j]);
        }
        return wave_reduce(acc, op);
    }
};

// ---- contiguous lines that fit one tile: one workgroup per line, no communication ------------------------
template <typename In, typename T, typename Out, typename Op, bool VECTOR, int K, int NW = 4>
__global__ __launch_bounds__(NW * WAVE) void scan_tiles_kernel(const In* __restrict__ in, Out* __restrict__ out, int64_t line_len, T init,
                                                         int inclusive, Op op) {
    __shared__ T lds_wave[NW];
    const T ident = Op::template identity<T>();
    const int wave = threadIdx.x / WAVE;
    const int64_t e0 = (int64_t)blockIdx.x * line_len;
    TileRegs<T, K> r;
    const T wtot = tile_load_scan<In, T, Op, VECTOR, K, NW>(in, e0, (int)line_len, inclusive, op, r);
    if (lane_id() == 0) lds_wave[wave] = wtot;
    __syncthreads();
    T wave_prefix = ident;
#pragma unroll
    for (int w = 0; w < NW; ++w)
        if (w < wave) wave_prefix = op(wave_prefix, lds_wave[w]);
    tile_store<Out, T, Op, VECTOR, K, NW>(out, e0, (int)line_len, op(init, wave_prefix), op, r);
}

// ---- long contiguous lines: persistent workgroups, single pass, two-level decoupled look-back --------------
// `counter` packs (epoch << 32 | acquisitions).  A workgroup takes its tiles from it in acquisition order:
// every predecessor of a tile is therefore already owned by a running workgroup, so the look-back never
// waits on work that has not started.  The id of the next tile is taken only when the workgroup is ready
// to load it -- ids taken ahead of time would be published late and stall every successor.
// Device-wide atomics on one address complete at about 14 ns each on MI355X, so the tile is made as large
// as the problem allows (up to 1024 threads x 8 vectors = 128 KiB of input): 2^27 elements are 4096
// acquisitions, ~60 us, against ~170 us of streaming.
constexpr int SCAN_SWEEP = 1024;

// Every workgroup of a chained kernel makes exactly one acquisition beyond the last tile, so acquisition number
// ntiles + gridDim.x - 1 is the last access of the call.  Its owner (wave 0 runs this) advances the epoch and
// resets the count for the next call, and clears a rotating slice of the descriptor slots this call did not
// use, so that no slot keeps a tag for more than SCAN_SWEEP calls (tags are 30-bit epochs).
__device__ __forceinline__ void chain_finish(unsigned long long cur, int64_t ntiles, int64_t used, unsigned long long* counter,
                                             uint64_t* desc, int64_t desc_capacity) {
    if (threadIdx.x >= WAVE || (int64_t)(cur & 0xffffffffull) != ntiles + (int64_t)gridDim.x - 1) return;
    const int lane = lane_id();
    uint32_t epoch = (uint32_t)(cur >> 32);
    const int64_t slice = (desc_capacity + SCAN_SWEEP - 1) / SCAN_SWEEP;
    int64_t lo = (int64_t)(epoch % SCAN_SWEEP) * slice, hi = lo + slice;
    if (lo < used) lo = used;
    if (hi > desc_capacity) hi = desc_capacity;
    for (int64_t i = lo + lane; i < hi; i += WAVE) desc[i] = 0;
    epoch = (epoch + 1u) & 0x3fffffffu;
    if (epoch == 0u) epoch = 1u;          // tag 0 marks a cleared slot
    if (lane == 0) *counter = (unsigned long long)epoch << 32;
}

template <typename In, typename T, typename Out, typename Op, bool VECTOR, int K, int NW>
__global__ __launch_bounds__(NW * WAVE) void scan_chain_kernel(const In* __restrict__ in, Out* __restrict__ out, int64_t line_len,
                                                         int64_t tiles_per_line, int64_t ntiles, T init, int inclusive, Op op,
                                                         unsigned long long* counter, uint64_t* desc, int64_t ngroups_per_line,
                                                         int64_t ngroups, int64_t desc_capacity, WaitCtl wc) {
    constexpr int VEC = 16 / sizeof(T);
    constexpr int TILE = NW * WAVE * VEC * K;
    __shared__ T lds_wave[NW];
    __shared__ T lds_prefix;
    __shared__ unsigned long long lds_id;

    const T ident = Op::template identity<T>();
    const int tid = threadIdx.x, wave = tid / WAVE, lane = lane_id();
    uint64_t* tile_desc = desc;                                        // [words][ntiles]
    uint64_t* group_desc = desc + (int64_t)Words<T>::N * ntiles;       // [words][ngroups]

    if (tid == 0) lds_id = __hip_atomic_fetch_add(counter, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    unsigned long long cur = lds_id;
    while ((int64_t)(cur & 0xffffffffull) < ntiles) {
        const int64_t tile = (int64_t)(cur & 0xffffffffull);
        const uint32_t epoch = (uint32_t)(cur >> 32);
        wc.stamp = epoch;
        const int64_t line = tile / tiles_per_line, tl = tile - line * tiles_per_line;
        const int64_t e0 = line * line_len + tl * TILE;
        const int64_t left = line_len - tl * TILE;
        const int valid = left < TILE ? (int)left : TILE;
        TileRegs<T, K> r;
        const T wtot = tile_load_scan<In, T, Op, VECTOR, K, NW>(in, e0, valid, inclusive, op, r);
        if (lane == 0) lds_wave[wave] = wtot;
        __syncthreads();
        T wave_prefix = ident, tile_agg = ident;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const T x = lds_wave[w];
            if (w < wave) wave_prefix = op(wave_prefix, x);
            tile_agg = op(tile_agg, x);
        }
        if (wave == 0) {
            T tile_prefix = init;
            if (lane == 0) desc_publish(tile_desc, ntiles, tile, tile_agg, (epoch << 2) | DESC_A);
            if (tl > 0)
                tile_prefix = desc_lookback2(tile_desc, ntiles, group_desc, ngroups, tile, tl, line * ngroups_per_line + (tl >> 6),
                                             epoch, tile_agg, init, op, ident, wc);
            if (lane == 0) lds_prefix = tile_prefix;
        }
        __syncthreads();
        tile_store<Out, T, Op, VECTOR, K, NW>(out, e0, valid, op(lds_prefix, wave_prefix), op, r);
        if (tid == 0) lds_id = __hip_atomic_fetch_add(counter, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        cur = lds_id;
    }
    chain_finish(cur, ntiles, (int64_t)Words<T>::N * (ntiles + ngroups), counter, desc, desc_capacity);
}

// The tile of a workgroup of an "ordered" kernel (one tile per workgroup, every tile waits only for tiles of lower
// number) and the epoch of the call.  dynamic_ids == 0: the workgroup's index.  Workgroups are dealt to the XCDs
// round-robin by index and every XCD starts its share in index order, so for ONE grid alone on the device the lowest
// unfinished tile is always resident and waits for nobody.  Across XCDs nothing orders the starts: tile 9 (XCD 1) may
// be resident and waiting while tile 8 (XCD 0) still waits for a slot, and with a second such grid resident the slots
// of XCD 0 may all be held by ITS waiting tiles, whose own lowest unfinished tile waits for a slot on XCD 1: a cycle
// that no arbitration rule of the hardware is known to exclude.  Hence a kernel runs in launch order only where that
// cannot happen -- its tiles help themselves when a wait drags on (desc_lookback_alone), or a tile waits only for
// tiles of its own XCD -- and otherwise takes its tile numbers from the packed counter (dynamic_ids != 0; one
// device-wide atomic per workgroup, which returns the epoch with the number; 8-10 % slower, the round trip sits in
// front of every tile's loads, and neither asking for the next number behind the stores nor during the look-back of
// the tile before hid it: 2^26 Int32 90 -> 100 / 104 / 112 us): a tile's predecessors then belong to workgroups that
// have started, whatever else is resident.  Grids that fit the device whole stay in launch order.
// `need_epoch` (wave-uniform): this wave uses the epoch -- the others of a launch-order grid skip the load and get 0.
struct OrderedId { int64_t tile; uint32_t epoch; };
__device__ __forceinline__ OrderedId ordered_tile_id(unsigned long long* counter, int dynamic_ids, bool need_epoch) {
    __shared__ unsigned long long lds_ordered_id;
    if (dynamic_ids == 0)
        return OrderedId{(int64_t)blockIdx.x,
                         need_epoch ? (uint32_t)(__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 32) : 0u};
    if (threadIdx.x == 0) lds_ordered_id = __hip_atomic_fetch_add(counter, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const unsigned long long cur = lds_ordered_id;
    return OrderedId{(int64_t)(cur & 0xffffffffull), (uint32_t)(cur >> 32)};
}

// End of a kernel whose workgroups read the epoch from the header instead of acquiring it: the workgroup that leaves
// last (two levels of exit tickets: groups of `ticket_group` workgroups share a first-level ticket, each ticket on
// its own 128-byte line) advances the epoch and clears a rotating slice of the descriptor slots this call did not
// use, like chain_finish.  Every workgroup has read the epoch before it leaves, so nobody can see the new one.
__device__ __forceinline__ void ordered_finish(uint32_t epoch, int64_t used, unsigned long long* counter, uint32_t* tickets,
                                               int ticket_group, uint64_t* desc, int64_t desc_capacity) {
    __shared__ int lds_last;
    const int tid = threadIdx.x;
    if (tid == 0) {
        const int64_t nb = gridDim.x, ng = (nb + ticket_group - 1) / ticket_group, grp = blockIdx.x / ticket_group;
        const uint32_t gsize = (uint32_t)(grp == ng - 1 ? nb - grp * ticket_group : ticket_group);
        int last = 0;
        uint32_t* gt = tickets + grp * TICKET_STRIDE;
        if (__hip_atomic_fetch_add(gt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gsize - 1u) {
            *gt = 0;                                                            // clean for the next call
            uint32_t* lt = tickets + ng * TICKET_STRIDE;
            if (__hip_atomic_fetch_add(lt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (uint32_t)ng - 1u) {
                *lt = 0;
                last = 1;
            }
        }
        lds_last = last;
    }
    __syncthreads();
    if (!lds_last || tid >= WAVE) return;
    const int lane = lane_id();
    const int64_t slice = (desc_capacity + SCAN_SWEEP - 1) / SCAN_SWEEP;
    int64_t lo = (int64_t)(epoch % SCAN_SWEEP) * slice, hi = lo + slice;
    if (lo < used) lo = used;
    if (hi > desc_capacity) hi = desc_capacity;
    for (int64_t i = lo + lane; i < hi; i += WAVE) desc[i] = 0;
    uint32_t e = (epoch + 1u) & 0x3fffffffu;
    if (e == 0u) e = 1u;                  // tag 0 marks a cleared slot
    if (lane == 0) *counter = (unsigned long long)e << 32;
}
// Workgroups of `threads` threads that an ordered kernel (compiled for 8 waves per SIMD, a few hundred bytes of LDS) has
// resident at once, and whether a grid of `nblocks` takes its tile numbers from the counter (see ordered_tile_id).
int tune_ordered_ids();            // rk_api.hip: 0 = by grid size, 1 = always the launch order, 2 = always the counter
inline int64_t ordered_resident(int threads) { return (int64_t)device_info().cus * (32 * WAVE / threads); }
// `launch_order_safe`: the launch order cannot starve the grid whatever else is resident -- the kernel's waits end in
// desc_lookback_alone, so its tiles need nobody; or every tile waits only for tiles of its own XCD (see
// rows_chains_stay_on_their_xcd).
inline int ordered_dynamic_ids(int64_t nblocks, int threads, bool launch_order_safe) {
    const int t = tune_ordered_ids();
    return t == 1 ? 0 : (t == 2 ? 1 : (!launch_order_safe && nblocks > ordered_resident(threads) ? 1 : 0));
}
// The scans across rows number their tiles slice-major: tile = slice * nchains + chain, and a tile waits only for tiles
// of its own chain.  Workgroups are dealt to the XCDs round-robin by index and each XCD starts its share in index order.
// With the number of chains a multiple of 8 (of the number of XCDs, which divides 8) all tiles of a chain fall to one
// XCD, so a resident tile waits only for tiles that the same XCD has started before it: the lowest resident tile of an
// XCD waits for nobody, finishes, and so on up -- every resident tile finishes without any new workgroup having to
// start, whatever other grids hold the remaining slots.  Other chain counts take their tile numbers from the counter.
inline bool rows_chains_stay_on_their_xcd(int64_t nchains) { return nchains % 8 == 0; }
// Workgroups per first-level exit ticket: at most half of the ticket lines in use, at least TICKET_GROUP a ticket.
inline int ordered_ticket_group(int64_t nblocks) {
    int64_t tg = (nblocks + (int64_t)WS_TICKET_COUNT / 2 - 1) / ((int64_t)WS_TICKET_COUNT / 2);
    return (int)(tg < TICKET_GROUP ? TICKET_GROUP : tg);
}

// ---- long contiguous lines: one tile per workgroup in launch order, single pass ------------------------------------
// Tile = blockIdx.x.  No tile counter: device-wide atomics on one address complete at about 14 ns each, and the
// counter's round trip would sit in front of every tile's loads (2^26 Int32: 90 -> 100 us).  Forward progress does not
// rest on the order in which workgroups start: a tile that has polled `wa.patience` times in vain stops waiting and
// resolves its prefix alone, computing the aggregates nobody has published from the input (desc_lookback_alone), so
// no tile needs another workgroup to be running.  Wave 0 parks its part of the tile in LDS while it looks back, which
// leaves that path -- and the compiler -- the registers it needs.
// 1024 threads x 8 vectors = 128 KiB of input per tile at <= 64 registers: two workgroups share a compute unit, one
// loads or stores while the other waits for its prefix (at 112 registers and one workgroup per unit the wait was
// dead time: 2^26 Int32 95.6 -> 92.5 us, 2^27 187.8 -> 180.5 us).  Smaller tiles stream better on their own (16 KiB
// tiles without any look-back: 86 us) but lose more to the look-back than they gain.
// The epoch of the call is read from the workspace header; the workgroup that leaves last (two-level exit tickets)
// advances it and clears a rotating slice of unused descriptor slots, like chain_finish.
// Compiled for 8 waves per SIMD (<= 64 registers), for aligned lines.  8-byte values hold the same 32 registers of
// data but scan with twice the temporaries: their vectors are scanned strictly one after the other (tile_scan_regs),
// which keeps them inside the 64 registers (interleaved they spilled 20).
// PACKED: 1- and 2-byte integers stay packed in the registers (see Packed): the tile is 128 KiB of them, not 32 or 64.
template <typename In, typename T, typename Out, typename Op, bool VECTOR, int K, int NW, bool PACKED = false>
__global__ __launch_bounds__(NW * WAVE, 8) void scan_ordered_kernel(const In* __restrict__ in, Out* __restrict__ out, int64_t line_len,
                                                                    int64_t tiles_per_line, int64_t ntiles, T init, int inclusive, Op op,
                                                                    unsigned long long* counter, uint32_t* tickets, int ticket_group,
                                                                    uint64_t* desc, int64_t ngroups_per_line, int64_t ngroups,
                                                                    int64_t desc_capacity, WaitCtl wc, WaitAlone wa, int stagger_ticks, int stagger_tiles, int dynamic_ids) {
    constexpr int VEC = PACKED ? 16 / (int)sizeof(In) : 16 / (int)sizeof(T);    // elements per 16-byte register group
    constexpr int TILE = NW * WAVE * VEC * K;
    typedef typename std::conditional<PACKED, PackedRegs<K>, TileRegs<T, K>>::type Regs;
    typedef typename std::conditional<PACKED, PackedVec, typename VecOf<T, 16 / sizeof(T)>::type>::type VT;
    __shared__ T lds_wave[NW];
    __shared__ T lds_prefix;
    __shared__ VT lds_stash[K][WAVE];         // wave 0's registers while it resolves its prefix alone
    const T ident = Op::template identity<T>();
    const int tid = threadIdx.x, wave = tid / WAVE, lane = lane_id();
    uint64_t* tile_desc = desc;                                        // [words][ntiles]
    uint64_t* group_desc = desc + (int64_t)Words<T>::N * ntiles;       // [ngroups] lines
    const OrderedId id = ordered_tile_id(counter, dynamic_ids, wave == 0);      // wave 0 looks back and leaves last
    const uint32_t epoch = id.epoch;
    wc.stamp = epoch;
    // The workgroups of the first resident round start together, so they would load together, wait for their prefixes
    // together and store together, and the rounds behind them inherit the rhythm: memory idles while everybody waits.
    // Tile i of that round therefore starts i / stagger_tiles of `stagger_ticks` (100 MHz clock) late.
    if (id.tile < stagger_tiles) {
        const long long d = (long long)stagger_ticks * id.tile / stagger_tiles;
        const long long t0 = wall_clock64();
        while (wall_clock64() - t0 < d) __builtin_amdgcn_s_sleep(4);
    }
    {
        const int64_t tile = id.tile;
        const int64_t line = tile / tiles_per_line, tl = tile - line * tiles_per_line;
        const int64_t e0 = line * line_len + tl * TILE;
        const int64_t left = line_len - tl * TILE;
        const int valid = left < TILE ? (int)left : TILE;
        Regs r;
        T wtot;
        if constexpr (PACKED) wtot = packed_tile_load_scan<In, T, Op, K, NW>(in, e0, valid, inclusive, op, r);
        else wtot = tile_load_scan<In, T, Op, VECTOR, K, NW>(in, e0, valid, inclusive, op, r);
        if (lane == 0) lds_wave[wave] = wtot;
        __syncthreads();
        if (wave == 0) {
            static_assert(NW <= WAVE, "the wave totals are scanned by one wave");
            const T x = lane < NW ? lds_wave[lane] : ident;
            const T inc = wave_scan_inclusive(x, op, ident);
            const T tile_agg = read_lane(inc, NW - 1);
            if (lane < NW) lds_wave[lane] = wave_shift_right(inc, ident);       // what lies in front of each wave inside the tile
            T tile_prefix = init;
            if (lane == 0) desc_publish(tile_desc, ntiles, tile, tile_agg, (epoch << 2) | DESC_A);
            // a line's first tile has no look-back between this and its stores: the aggregate is out before them (a tile
            // that helps itself in an in-place scan counts on that order, see desc_sum_or_compute)
            if (tl == 0) publish_barrier();
            if (tl > 0) {
                // The wave's part of the tile waits in LDS while the wave looks back: the kernel is compiled for 64
                // registers, the tile takes 32 of them, and the way out of an endless wait (desc_lookback_alone, which
                // reads other tiles) needs more than the rest -- with the tile in registers the compiler made room in
                // private memory, inside the tile's scan.  Sixteen LDS accesses a tile, by one wave of sixteen.
                volatile VT* stash = &lds_stash[0][lane];
#pragma unroll
                for (int k = 0; k < K; ++k) stash[k * WAVE] = r.v[k];
                bool expired = false;
                const int64_t gl = line * ngroups_per_line + (tl >> 6);
                tile_prefix = desc_lookback_leader(tile_desc, ntiles, group_desc, tile, tl, gl, epoch, tile_agg, init, op, ident, wc, wa, expired);
                if (expired)
                    tile_prefix = desc_lookback_alone(tile_desc, ntiles, group_desc, tile, tl, gl, epoch, tile_agg, init, op, ident,
                                                      ScanTileAggregate<In, T, Op, TILE, VECTOR>{in + e0, tile}, wa.counter);
#pragma unroll
                for (int k = 0; k < K; ++k) r.v[k] = stash[k * WAVE];
            }
            if (lane == 0) lds_prefix = tile_prefix;
        }
        __syncthreads();
        if constexpr (PACKED) packed_tile_store<In, T, Op, K, NW>(out, e0, valid, op(lds_prefix, lds_wave[wave]), op, r);
        else tile_store<Out, T, Op, VECTOR, K, NW>(out, e0, valid, op(lds_prefix, lds_wave[wave]), op, r);
    }
    ordered_finish(epoch, (int64_t)Words<T>::N * ntiles + ngroups * GROUP_DESC_STRIDE, counter, tickets, ticket_group, desc, desc_capacity);
}

// ---- contiguous lines shorter than a tile: one wave per line -------------------------------------
// VECTOR: lines are whole 16-byte vectors at 16-byte aligned addresses.  Otherwise, for 4- and 8-byte elements, the lanes
// still take 16 bytes each -- global memory accepts that at any element-aligned address -- and only the vector the
// line's end cuts goes element by element (cumsum(A; dims=1) of 257 x 240000 Float32: 143 us with one element a
// lane, 100 us).
template <typename In, typename T, typename Out, typename Op, bool VECTOR, int BLOCK>
__global__ __launch_bounds__(BLOCK) void scan_wave_lines_kernel(const In* __restrict__ in, Out* __restrict__ out, int64_t line_len,
                                                                int64_t nlines, T init, int inclusive, Op op) {
    constexpr bool ELEMS = !VECTOR && ElemVectors<In, T>::value && OutElemVectors<Out, T>::value;        // vectors at element-aligned addresses
    constexpr int VEC = (VECTOR || ELEMS) ? 16 / sizeof(T) : 1;
    typedef typename VecOf<T, VEC>::type VT;
    typedef typename VecOf<In, VEC>::type VI;
    const int64_t line = (int64_t)blockIdx.x * (BLOCK / WAVE) + threadIdx.x / WAVE;
    if (line >= nlines) return;
    const int lane = lane_id();
    const T ident = Op::template identity<T>();
    const int64_t base = line * line_len;
    T carry = init;
    for (int64_t c = 0; c < line_len; c += WAVE * VEC) {
        const int64_t i0 = c + (int64_t)lane * VEC;
        const bool whole = i0 + VEC <= line_len;               // VECTOR: line_len % VEC == 0, a vector is inside or outside
        T v[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = ident;
        if constexpr (VEC == 1) {
            if (whole) v[0] = (T)in[base + i0];
        } else {
            if (whole) {
                VI x;
                if constexpr (ELEMS) x = ElemVectors<In, T>::template load<VEC>(in + base + i0);
                else x = load_nt((const VI*)(in + base + i0));
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[j] = (T)x[j];
            } else if (ELEMS && i0 < line_len) {
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    if (i0 + j < line_len) v[j] = (T)in[base + i0 + j];
            }
        }
#pragma unroll
        for (int j = 1; j < VEC; ++j) v[j] = op(v[j - 1], v[j]);
        const T inc = wave_scan_inclusive(v[VEC - 1], op, ident);
        const T off = op(carry, wave_shift_right(inc, ident));
        carry = op(carry, read_lane(inc, WAVE - 1));
        if (i0 < line_len) {
            if constexpr (VEC == 1) {
                out[base + i0] = (Out)(inclusive ? op(off, v[0]) : off);
            } else {
                VT o;
                if (inclusive) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) o[j] = op(off, v[j]);
                } else {
                    o[0] = off;
#pragma unroll
                    for (int j = 1; j < VEC; ++j) o[j] = op(off, v[j - 1]);
                }
                if (whole) {
                    if constexpr (ELEMS) out_store_elems<Out, T, VEC>(out + base + i0, o);
                    else out_store_nt<Out, T, VEC>(out + base + i0, o);
                } else {
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        if (i0 + j < line_len) out[base + i0 + j] = (Out)o[j];
                }
            }
        }
    }
}

// ---- one lane per line (tiny lines, or narrow `inner`) ---------------------------------------------
template <typename In, typename T, typename Out, typename Op, int BLOCK>
__global__ __launch_bounds__(BLOCK) void scan_thread_kernel(const In* __restrict__ in, Out* __restrict__ out, ScanGeom g, T init,
                                                            int inclusive, Op op) {
    const int64_t line = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (line >= g.inner * g.outer) return;
    const int64_t o = line / g.inner, i = line - o * g.inner;
    const int64_t base = i + o * g.inner * g.mid;
    T acc = init;
    for (int64_t m = 0; m < g.mid; ++m) {
        const T x = (T)in[base + m * g.inner];
        if (inclusive) { acc = op(acc, x); out[base + m * g.inner] = (Out)acc; }
        else { out[base + m * g.inner] = (Out)acc; acc = op(acc, x); }
    }
}

// ---- short contiguous lines: a group of lanes per line, one 16-byte vector per lane ------------------------------
// (line length a multiple of the vector and at most 32 vectors, 16-byte aligned).  Lane l of a wave takes vector l of
// the wave's chunk, so loads and stores are fully coalesced whatever the line length; line = l / L, position = l % L
// with L vectors per line, and the 64 % L lanes past the last whole line idle.  Each lane scans its vector, the
// vector totals are scanned over the lanes of the line by shuffles that never cross a line start.  One lane per
// line with whole vectors reaches 1 TB/s on the same shape, one lane per line with scalars half of that
// (cumsum of 16 x 1_000_000 Float32 along dim 1: 231 us -> 128 us -> 42 us).
template <typename In, typename T, typename Out, typename Op, int BLOCK>
__global__ __launch_bounds__(BLOCK) void scan_short_lines_kernel(const In* __restrict__ in, Out* __restrict__ out, int L, int64_t nlines,
                                                                 T init, int inclusive, Op op) {
    constexpr int VEC = 16 / sizeof(T), U = 4;
    typedef typename VecOf<In, VEC>::type VI;
    typedef typename VecOf<T, VEC>::type VT;
    const int lane = threadIdx.x & 63;
    const int lpw = 64 / L;                                  // whole lines per wave and step
    const int ln = lane / L, pos = lane - ln * L;
    const int64_t wave_id = (int64_t)blockIdx.x * (BLOCK / 64) + (threadIdx.x >> 6);
    VI x[U];
    bool live[U];
    int64_t vecidx[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t line = (wave_id * U + u) * lpw + ln;
        live[u] = ln < lpw && line < nlines;
        vecidx[u] = line * L + pos;
        // unconditional: a load under a branch of its own is waited for before the next one is issued; lanes without
        // a line read vector 0 (nlines > 0) and drop it
        x[u] = load_nt((const VI*)in + (live[u] ? vecidx[u] : 0));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        T loc[VEC];
        loc[0] = (T)x[u][0];
#pragma unroll
        for (int j = 1; j < VEC; ++j) loc[j] = op(loc[j - 1], (T)x[u][j]);
        T tot = loc[VEC - 1];
        for (int d = 1; d < L; d <<= 1) {
            const T v = __shfl_up(tot, d, 64);
            if (pos >= d) tot = op(v, tot);
        }
        const T prev = __shfl_up(tot, 1, 64);
        const T base = pos > 0 ? op(init, prev) : init;
        VT o;
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[j] = inclusive ? op(base, loc[j]) : (j == 0 ? base : op(base, loc[j > 0 ? j - 1 : 0]));
        if (live[u]) out_store_nt<Out, T, VEC>(out + vecidx[u] * VEC, o);
    }
}

// ---- short lines of any length, contiguous or with a narrow inner extent: whole slabs through LDS -----------------
// (cumsum(A; dims=1) of a 15 x 2_000_000 array: the line length is no multiple of the 16-byte vector, so lines start
// at odd addresses; a lane per line reads with a stride of 60 bytes -- 425 us -- and a wave per line idles 49 lanes.
// cumsum(A; dims=2) of a 4 x 32 x 250_000 array: a lane per line walks 32 rows of 16 bytes.)
// A slab is the inner x mid block of one outer index, contiguous in memory.  A workgroup copies a 16 KiB run of whole
// slabs into LDS with 16-byte loads (the host picks the slabs per block so that every block starts at a whole vector),
// a group of tpl = 1, 2 .. 64 lanes scans each line in place -- lane `part` owns a segment of ceil(m / tpl) elements,
// the segment totals are scanned over the group's lanes by shuffles that never cross a group -- and the tile leaves
// with 16-byte stores.
constexpr int SCAN_LDS_LINES_MAX = 128;     // contiguous lines beyond, and whole vectors beyond 64: a wave per line does as well or better

template <typename In, typename T, typename Out, typename Op, bool VECTOR>
__global__ __launch_bounds__(256) void scan_lds_lines_kernel(const In* __restrict__ in, Out* __restrict__ out, int inner, int m, int64_t nslabs,
                                                             int slabs_per_block, int tpl_log2, T init, int inclusive, Op op) {
    constexpr int TE = 16384 / sizeof(T);
    __shared__ __attribute__((aligned(16))) T lds[TE];
    const int t = threadIdx.x;
    const int slab = inner * m;
    const int64_t slab0 = (int64_t)blockIdx.x * slabs_per_block;
    const int64_t left = nslabs - slab0;
    const int ns = left < slabs_per_block ? (int)left : slabs_per_block;     // > 0 by the grid size
    const int ne = ns * slab;                                                 // <= TE by the choice of slabs_per_block
    const In* p = in + slab0 * slab;
    Out* q = out + slab0 * slab;
    constexpr int VEC = VECTOR ? 16 / sizeof(T) : 1;
    typedef typename VecOf<In, VEC>::type VI;
    typedef typename VecOf<T, VEC>::type VT;
    const int nv = ne / VEC;
    if constexpr (VEC == 1) {
        for (int i = t; i < nv; i += 256) lds[i] = (T)p[i];
    } else {
        // at most TE / VEC / 256 = 4 vectors a thread: all loads issued before the first LDS write, and none under a
        // branch of its own (such a load is waited for before the next one is issued): past the end, vector 0 again
        constexpr int ROUNDS = TE / VEC / 256;
        VI v[ROUNDS];
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) v[r] = nv > 0 ? load_nt((const VI*)p + (t + r * 256 < nv ? t + r * 256 : 0)) : VI{};   // nv: uniform
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
            if (t + r * 256 < nv) {
                VT w;
#pragma unroll
                for (int j = 0; j < VEC; ++j) w[j] = (T)v[r][j];
                ((VT*)lds)[t + r * 256] = w;
            }
        }
    }
    for (int e = nv * VEC + t; e < ne; e += 256) lds[e] = (T)p[e];           // fewer than VEC elements
    __syncthreads();
    const int tpl = 1 << tpl_log2;
    // an odd segment length: the lanes of a group start inner * seg elements apart, and an even pitch folds them onto
    // few banks (2 x 1000 x 16777 Float32 with 64 lanes a line: segments of 16 put 32 lanes on one bank, 234 us; of 17, 51 us)
    const int seg = ((m + tpl - 1) >> tpl_log2) | 1;
    const int nl = ns * inner;
    const int items = nl << tpl_log2;
    for (int base = 0; base < items; base += 256) {       // uniform trip count: the shuffles below need every lane
        const int idx = base + t;
        const int l = idx >> tpl_log2, part = idx & (tpl - 1);
        const int k0 = part * seg;
        const int k1 = k0 + seg < m ? k0 + seg : m;
        const bool live = l < nl && k0 < m;                // empty segments sit at the end of a group: nothing reads them
        const int sl = live ? l / inner : 0;
        T* line = lds + (live ? sl * slab + (l - sl * inner) : 0);
        if (tpl_log2 == 0) {
            // a lane per line: one sweep, init folded in
            if (live) {
                T run = init;
                if (inclusive) {
                    for (int k = 0; k < m; ++k) { run = op(run, line[k * inner]); line[k * inner] = run; }
                } else {
                    for (int k = 0; k < m; ++k) { const T x = line[k * inner]; line[k * inner] = run; run = op(run, x); }
                }
            }
            continue;
        }
        T tot = init;
        if (live) {
            tot = line[k0 * inner];
            for (int k = k0 + 1; k < k1; ++k) {
                tot = op(tot, line[k * inner]);
                line[k * inner] = tot;
            }
        }
        for (int d = 1; d < tpl; d <<= 1) {
            const T v = __shfl_up(tot, d, 64);
            if (part >= d) tot = op(v, tot);
        }
        const T prev = __shfl_up(tot, 1, 64);
        const T before = part > 0 ? op(init, prev) : init;
        if (live) {
            if (inclusive) {
                for (int k = k0; k < k1; ++k) line[k * inner] = op(before, line[k * inner]);
            } else {
                for (int k = k1 - 1; k > k0; --k) line[k * inner] = op(before, line[(k - 1) * inner]);
                line[k0 * inner] = before;
            }
        }
    }
    __syncthreads();
    if constexpr (VEC == 1) {
        for (int i = t; i < nv; i += 256) q[i] = (Out)lds[i];
    } else {
        constexpr int ROUNDS = TE / VEC / 256;
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r)
            if (t + r * 256 < nv) out_store_nt<Out, T, VEC>(q + (t + r * 256) * VEC, ((const VT*)lds)[t + r * 256]);
    }
    for (int e = nv * VEC + t; e < ne; e += 256) q[e] = (Out)lds[e];
}

// ---- 1 < inner < 64 with long lines: tiles of whole rows through LDS ----------------------------------
// Lanes along `inner` would leave most of a wave idle, and one lane per line (scan_thread_kernel) walks the line
// alone.  Here a workgroup takes a tile of consecutive rows -- contiguous memory, loaded and stored coalesced --
// into LDS.  Thread t owns column t % inner and the (t / inner)-th segment of the tile's rows; neighbouring threads
// touch neighbouring LDS words.  Pass TOTALS: column totals of every tile.  After an exclusive scan of the totals
// along the tiles (seeded with init) the second pass scans every tile from its carried-in prefix.
// grid (tiles, outer); totals / carry: [(o * tiles + tile) * inner + column]; carry == nullptr: every column starts
// from `init` (a single tile per outer index).  VECTOR: every tile starts at a whole 16-byte vector of `out` (the host
// makes rows_per_tile * inner a multiple of the vector): the tile moves with 16-byte accesses, all loads of a thread
// issued before the first LDS write.  (One 4-byte load a loop step, each waited for before the next was issued:
// accumulate(+, 7 x 4_194_304 Float32; dims=2) 62 + 96 us for the two passes, now 24 + 46.)  `in` may be `out` (a tile is in LDS whole before any of it is written).
template <typename T> struct NarrowTile { static constexpr int ELEMS = sizeof(T) >= 8 ? 4096 : 8192; };

template <typename In, typename T, typename Out, typename Op, bool TOTALS, bool VECTOR>
__global__ __launch_bounds__(256) void scan_narrow_kernel(const In* in, Out* out, ScanGeom g, int inclusive, Op op,
                                                          int64_t rows_per_tile, T* carry, T init) {
    constexpr int ELEMS = NarrowTile<T>::ELEMS;
    constexpr int VEC = 16 / sizeof(T), ROUNDS = ELEMS / VEC / 256;
    typedef typename VecOf<T, VEC>::type VT;
    typedef typename VecOf<In, VEC>::type VI;
    __shared__ __attribute__((aligned(16))) T tile[ELEMS];
    __shared__ T seg_total[256];
    const int tid = threadIdx.x;
    const int inner = (int)g.inner;
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_tile;
    const int nrows = (int)(r0 + rows_per_tile <= g.mid ? rows_per_tile : g.mid - r0);
    const int count = nrows * inner;
    const int64_t base = (int64_t)blockIdx.y * g.inner * g.mid + r0 * g.inner;
    const int nv = VECTOR ? count / VEC : 0;                       // whole vectors of the tile
    if (VECTOR && nv > 0) {
        // every thread issues all its loads, the ones past the end re-reading the tile's last vector: a load under a
        // branch of its own is waited for before the next one is issued (eight memory round trips instead of one)
        VI x[ROUNDS];
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
            const int i = tid + r * 256;
            x[r] = load_nt((const VI*)(in + base) + (i < nv ? i : nv - 1));
        }
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r)
            if (tid + r * 256 < nv) {
                VT y;
#pragma unroll
                for (int j = 0; j < VEC; ++j) y[j] = (T)x[r][j];
                ((VT*)tile)[tid + r * 256] = y;
            }
    }
    for (int e = nv * VEC + tid; e < count; e += 256) tile[e] = (T)in[base + e];
    __syncthreads();
    const int nseg = 256 / inner;                                  // segments of rows per column
    const int c = tid % inner, sgm = tid / inner;
    const bool active = sgm < nseg;
    const int seg_rows = (nrows + nseg - 1) / nseg;
    const int row_lo = sgm * seg_rows, row_hi = row_lo + seg_rows < nrows ? row_lo + seg_rows : nrows;
    const T ident = Op::template identity<T>();
    // LDS is read in batches of independent loads instead of one load a step, each waited for (worth 1 .. 6 %:
    // 7 x 4_194_304 Float32 89 -> 84 us, 3 x 1_000_000 Int64 31 -> 29 us).
    constexpr int B = 8;
    T tot = ident;
    if (active) {
#pragma unroll 1
        for (int r = row_lo; r < row_hi; r += B) {
            T v[B];
#pragma unroll
            for (int u = 0; u < B; ++u) v[u] = r + u < row_hi ? tile[(r + u) * inner + c] : ident;
#pragma unroll
            for (int u = 0; u < B; ++u) tot = op(tot, v[u]);
        }
    }
    seg_total[tid] = tot;                                          // index sgm * inner + c == tid for active threads
    __syncthreads();
    const int64_t slot = ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * inner + c;
    // the segments in front of this thread's (TOTALS: all segments, by the threads of segment 0), in order
    const int nfront = TOTALS ? (sgm == 0 ? nseg : 0) : sgm;
    T front = ident;
    if (active) {
#pragma unroll 1
        for (int q = 0; q < nfront; q += B) {
            T v[B];
#pragma unroll
            for (int u = 0; u < B; ++u) v[u] = q + u < nfront ? seg_total[(q + u) * inner + c] : ident;
#pragma unroll
            for (int u = 0; u < B; ++u) front = op(front, v[u]);
        }
    }
    if constexpr (TOTALS) {
        if (active && sgm == 0) carry[slot] = front;
    } else {
        if (active) {
            T run = op(carry != nullptr ? carry[slot] : init, front);
#pragma unroll 1
            for (int r = row_lo; r < row_hi; r += B) {
                T v[B];
#pragma unroll
                for (int u = 0; u < B; ++u) v[u] = r + u < row_hi ? tile[(r + u) * inner + c] : ident;
#pragma unroll
                for (int u = 0; u < B; ++u) {
                    const T nxt = op(run, v[u]);
                    if (r + u < row_hi) tile[(r + u) * inner + c] = inclusive ? nxt : run;
                    run = nxt;
                }
            }
        }
        __syncthreads();
        if constexpr (VECTOR) {
#pragma unroll
            for (int r = 0; r < ROUNDS; ++r)
                if (tid + r * 256 < nv) out_store_nt<Out, T, VEC>(out + base + (tid + r * 256) * VEC, ((const VT*)tile)[tid + r * 256]);
        }
        for (int e = nv * VEC + tid; e < count; e += 256) out[base + e] = (Out)tile[e];
    }
}

// ---- inner >= 64: lanes along `inner`, 4 waves share the rows of a chunk -----------------------------
// grid (strips * outer, slices): the outer index shares the x axis with the strips (the other axes end at 65535).
// A workgroup scans the rows [slice * rows_per_slice, +rows_per_slice) of its
// 64 * VEC columns: a wave keeps R consecutive rows in registers, scans them downwards, and the four waves
// exchange their column totals through LDS.  With one slice the scan starts from `init`; with several, the
// exclusive prefix of every (slice, column) comes from `carry_in` (scan_strided_totals_kernel + a scan of the
// totals), which makes the slices independent: 12 instead of 8 bytes per element, but thousands of workgroups
// instead of one per strip.
template <typename In, typename T, typename Out, typename Op, bool VECTOR, int R>
__global__ __launch_bounds__(256) void scan_strided_kernel(const In* __restrict__ in, Out* __restrict__ out, ScanGeom g, T init,
                                                           int inclusive, Op op, int64_t rows_per_slice,
                                                           const T* __restrict__ carry_in, int64_t carry_pitch, int64_t strips) {
    constexpr int VEC = VECTOR ? 16 / sizeof(T) : 1;
    constexpr int COLS = WAVE * VEC;
    constexpr int NW = 4;
    typedef typename VecOf<T, VEC>::type VT;
    typedef typename VecOf<In, VEC>::type VI;
    __shared__ T lds[NW][COLS];
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int64_t o = (int64_t)blockIdx.x / strips, strip = (int64_t)blockIdx.x - o * strips;
    // 4- and 8-byte elements: vectors at any element-aligned address, so rows need be no whole number of vectors.  The
    // last vector of such a row starts VEC elements before the row's end instead of running into the next row: its
    // leading columns are scanned, and stored, by the lane before as well, with the same values.  Column totals are
    // kept per lane slot (`nominal`), which is the column for every other lane.
    constexpr bool ANY_ALIGN = VECTOR && sizeof(In) >= 4 && OutElemVectors<Out, T>::value;
    const int64_t nominal = strip * COLS + (int64_t)lane * VEC;
    const bool live = nominal < g.inner;
    const int64_t col0 = (ANY_ALIGN && live && nominal + VEC > g.inner) ? g.inner - VEC : nominal;
    const int64_t slab = o * g.inner * g.mid;
    // (Running the slices last to first, so that the scan starts with what the totals pass read last, changed nothing.)
    const int64_t slice = (int64_t)blockIdx.y;
    const int64_t m_begin = slice * rows_per_slice;
    const int64_t m_end = m_begin + rows_per_slice < g.mid ? m_begin + rows_per_slice : g.mid;
    const T ident = Op::template identity<T>();
    T carry[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        carry[j] = (carry_in != nullptr && live) ? carry_in[(o * gridDim.y + slice) * carry_pitch + nominal + j] : init;
    for (int64_t m0 = m_begin; m0 < m_end; m0 += NW * R) {
        const int64_t row0 = m0 + (int64_t)wave * R;
        T v[R][VEC];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (live && row0 + r < m_end) {
                VI x;
                if constexpr (ANY_ALIGN) x = load_nt_elems<In, VEC>(in + slab + (row0 + r) * g.inner + col0);
                else x = load_nt((const VI*)(in + slab + (row0 + r) * g.inner + col0));
                if constexpr (VEC == 1) v[r][0] = (T)x;
                else {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) v[r][j] = (T)x[j];
                }
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[r][j] = ident;
            }
        }
#pragma unroll
        for (int r = 1; r < R; ++r)
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[r][j] = op(v[r - 1][j], v[r][j]);
#pragma unroll
        for (int j = 0; j < VEC; ++j) lds[wave][lane * VEC + j] = v[R - 1][j];
        __syncthreads();
        T pre[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            pre[j] = carry[j];
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const T x = lds[w][lane * VEC + j];
                if (w < wave) pre[j] = op(pre[j], x);
                carry[j] = op(carry[j], x);
            }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (live && row0 + r < m_end) {
                VT o;
                if constexpr (VEC == 1) o = inclusive ? op(pre[0], v[r][0]) : (r == 0 ? pre[0] : op(pre[0], v[r - 1][0]));
                else {
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        o[j] = inclusive ? op(pre[j], v[r][j]) : (r == 0 ? pre[j] : op(pre[j], v[r - 1][j]));
                }
                if constexpr (ANY_ALIGN) out_store_elems<Out, T, VEC>(out + slab + (row0 + r) * g.inner + col0, o);
                else out_store_nt<Out, T, VEC>(out + slab + (row0 + r) * g.inner + col0, o);
            }
        }
    }
}

// Column totals of every (slice, column): totals[(o * slices + slice) * pitch + column].
template <typename In, typename T, typename Op, bool VECTOR, int UNROLL>
__global__ __launch_bounds__(256) void scan_strided_totals_kernel(const In* __restrict__ in, T* __restrict__ totals, ScanGeom g, Op op,
                                                                  int64_t rows_per_slice, int64_t pitch, int64_t strips) {
    constexpr int VEC = VECTOR ? 16 / sizeof(T) : 1;
    constexpr int COLS = WAVE * VEC;
    constexpr int NW = 4;
    typedef typename VecOf<In, VEC>::type VI;
    __shared__ T lds[NW][COLS];
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int64_t o = (int64_t)blockIdx.x / strips, strip = (int64_t)blockIdx.x - o * strips;
    constexpr bool ANY_ALIGN = VECTOR && sizeof(In) >= 4 && sizeof(T) >= 4;     // as in scan_strided_kernel
    const int64_t nominal = strip * COLS + (int64_t)lane * VEC;
    const bool live = nominal < g.inner;
    const int64_t col0 = (ANY_ALIGN && live && nominal + VEC > g.inner) ? g.inner - VEC : nominal;
    const int64_t slab = o * g.inner * g.mid;
    auto load_row = [](const In* q) -> VI {
        if constexpr (ANY_ALIGN) return load_elems<In, VEC>(q);
        else return *(const VI*)q;
    };
    const int64_t m_begin = (int64_t)blockIdx.y * rows_per_slice;
    const int64_t m_end = m_begin + rows_per_slice < g.mid ? m_begin + rows_per_slice : g.mid;
    T acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = Op::template identity<T>();
    if (live) {
        // wave w takes the rows of its quarter of the slice in order (the same grouping as the scan kernel is
        // not required: only the totals matter, and they are combined in a fixed order).  Plain loads, not
        // non-temporal ones: the scan pass reads the same data next (4096 x 16384 Float32: 146 -> 136 us)
        int64_t m = m_begin + wave;
        for (; m + (UNROLL - 1) * NW < m_end; m += UNROLL * NW) {
            VI x[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) x[u] = load_row(in + slab + (m + u * NW) * g.inner + col0);
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                if constexpr (VEC == 1) acc[0] = op(acc[0], (T)x[u]);
                else {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) acc[j] = op(acc[j], (T)x[u][j]);
                }
            }
        }
        for (; m < m_end; m += NW) {
            const VI x = load_row(in + slab + m * g.inner + col0);
            if constexpr (VEC == 1) acc[0] = op(acc[0], (T)x);
            else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[j] = op(acc[j], (T)x[j]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) lds[wave][lane * VEC + j] = acc[j];
    __syncthreads();
    const int t = threadIdx.x;
    if (t < COLS) {
        T r = lds[0][t];
#pragma unroll
        for (int w = 1; w < NW; ++w) r = op(r, lds[w][t]);
        totals[(o * gridDim.y + blockIdx.y) * pitch + strip * COLS + t] = r;
    }
}

// ---- a short scanned dim behind a long contiguous one: a lane per group of columns ------------------------------
// (cumsum(A; dims=2) of a 50000 x 3 x 200 array: the strided kernel gives every workgroup three rows of a strip.)
// A lane owns VEC adjacent columns of one outer index and walks the <= 16 rows, loads four rows ahead; 16-byte accesses
// at element-aligned addresses, the last group of a row starting VEC columns before the row's end (it stores what the
// group before stores, the same values).  4- and 8-byte elements.
template <typename In, typename T, typename Out, typename Op>
__global__ __launch_bounds__(256) void scan_cols_kernel(const In* __restrict__ in, Out* __restrict__ out, ScanGeom g, T init, int inclusive,
                                                        Op op, int64_t groups_per_row, int64_t ngroups) {
    constexpr int VEC = 16 / sizeof(T);
    typedef typename VecOf<In, VEC>::type VI;
    typedef typename VecOf<T, VEC>::type VT;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= ngroups) return;
    const int64_t o = i / groups_per_row, q = i - o * groups_per_row;
    const int64_t col0 = q * VEC + VEC > g.inner ? g.inner - VEC : q * VEC;
    const int64_t base = o * g.inner * g.mid + col0;
    T run[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) run[j] = init;
    for (int64_t m0 = 0; m0 < g.mid; m0 += 4) {
        VI x[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) x[u] = ElemVectors<In, T>::template load<VEC>(in + base + (m0 + u < g.mid ? m0 + u : g.mid - 1) * g.inner);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (m0 + u < g.mid) {
                VT o4;
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const T nxt = op(run[j], (T)x[u][j]);
                    o4[j] = inclusive ? nxt : run[j];
                    run[j] = nxt;
                }
                out_store_elems<Out, T, VEC>(out + base + (m0 + u) * g.inner, o4);
            }
        }
    }
}

// ---- inner >= 64, few strips: tiles of rows in launch order, single pass --------------------------------------------
// scan_strided_kernel needs one workgroup per strip of 64 * VEC columns; a 4096 x 16384 matrix scanned along its rows
// has 16 strips.  Cutting the rows into slices makes the slices depend on each other.  The three-pass answer (column
// totals per slice, scan of the totals, scan from the carried-in prefix) reads the input twice: 12 bytes per element.
// Here a tile is NW * R = 150 rows of one strip and the dependency is resolved like in the single-pass scan of long lines,
// with a VECTOR for payload and two levels: a tile publishes its 64 * VEC column totals (1 KiB) and a flag, and sums
// the totals of its predecessors inside its group of ROWS_GROUP tiles; the last tile of a group publishes the group's
// aggregate; the first one (the leader) sums group aggregates back to the nearest published prefix and publishes the
// prefix through the previous group, which the other tiles of its group wait for.  With one level a tile read the
// totals of every tile in flight on its chain (32 KiB for 120 KiB of rows on a 4096 x 16384 matrix: 108 us); with two
// it reads 5 KiB on average.  Tiles are numbered slice-major (tile = slice * chains + chain, a chain
// being one strip of one outer index), so the workgroups in flight cover a compact band of whole rows and every
// predecessor has a lower blockIdx (forward progress as in scan_ordered_kernel).  HBM traffic: 8 bytes per element;
// the look-back reads one payload per tile in flight on the same chain -- a quarter of the tile's own bytes with 16
// chains -- from the device-coherent level, not from HBM.
//   flags     desc[tile]: tagged word, DESC_A = totals published; desc[ntiles + group]: DESC_A = aggregate of the
//             group published, DESC_P = inclusive prefix through the group published
//   payload   [ntiles + 2 * groups][64 * VEC] values in the partials area: totals; group aggregates; group prefixes
constexpr int ROWS_GROUP = 8;      // tiles of a chain per group of the two-level look-back

// The look-back of one tile (run by one wave): from the tile's column totals `tot` to `base`, the prefix of everything in
// front of the tile on its chain, `init` included.  Lane l holds the columns l * VEC .. l * VEC + VEC - 1.
// PACKED: only the first P * VEC columns are in use (P a power of two): the leader reads the aggregates of 64 / P groups
// with one load instruction, P lanes each, and folds them across the lanes, older ones on the left.  (All tiles of a
// long chain look back at the same time, so a leader walks every group in flight on the chain: 128 of them with
// 1024 tiles of one chain in flight, 32 round trips at four aggregates each.)
template <typename T, typename Op, int VEC, bool PACKED = false>
__device__ __forceinline__ void rows_lookback(const T (&tot)[VEC], T (&base)[VEC], T init, Op op, uint32_t epoch, int64_t tile, int64_t slice,
                                              int64_t chain, int64_t nchains, int64_t nslices, int64_t ntiles, T* payload, uint64_t* desc,
                                              const WaitCtl& wc, int lane, int P = WAVE) {
    constexpr int COLS = WAVE * VEC;
    typedef typename VecOf<T, VEC>::type VT;
    const T ident = Op::template identity<T>();
    const uint32_t tagA = (epoch << 2) | DESC_A, tagP = (epoch << 2) | DESC_P;
    const int64_t ngroups_chain = (nslices + ROWS_GROUP - 1) / ROWS_GROUP;
    uint64_t* gflag = desc + ntiles;                                    // [group * nchains + chain]
    T* gpayA = payload + ntiles * COLS;                                  // aggregates of whole groups
    T* gpayP = gpayA + ngroups_chain * nchains * COLS;                   // inclusive prefixes through a group
    const int r = (int)(slice % ROWS_GROUP);                             // predecessors inside the group
    const int64_t grp = slice / ROWS_GROUP;                              // groups in front of this one in the chain
#pragma unroll
    for (int j = 0; j < VEC; ++j) base[j] = init;
    const bool has_reader = slice + 1 < nslices;     // the last slice of a chain has none
    if (has_reader && r < ROWS_GROUP - 1) {          // the group's last tile publishes the group aggregate instead
        VT t;
#pragma unroll
        for (int j = 0; j < VEC; ++j) t[j] = tot[j];
        store_agent((VT*)(payload + tile * COLS + lane * VEC), t);
        publish_barrier();                           // the totals are at the coherent level before the flag
        if (lane == 0) __hip_atomic_store(&desc[tile], (uint64_t)tagA << 32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    long long rounds = 0;
    if (r == 0) {
        if (grp > 0) {
            // leader: aggregates of the groups in front, back to the nearest published prefix; publishes the
            // prefix through the previous group for the other tiles of its own
            T acc[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] = ident;
            int64_t first = grp - 1, rem = grp;
            for (;;) {
                uint32_t st = DESC_P;                // lanes beyond the first group: terminators
                if (lane < rem) {
                    const uint32_t tag = (uint32_t)(__hip_atomic_load(&gflag[(first - lane) * nchains + chain], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 32);
                    st = tag == tagA ? DESC_A : (tag == tagP ? DESC_P : 0u);
                }
                const uint64_t ballotP = __ballot(st == DESC_P);
                const uint64_t ballotX = __ballot(st == 0u);
                const int np = ballotP ? (__ffsll((unsigned long long)ballotP) - 1) : -1;
                const uint64_t needed = np >= 0 ? ((1ull << np) - 1ull) : ~0ull;
                if ((ballotX & needed) == 0ull) {
                    const int cnt = np >= 0 ? np : WAVE;
                    if constexpr (PACKED) {
                        constexpr int U = 4;
                        const int k = lane / P, pl = lane - k * P;          // lane pl of the k-th aggregate of a load
                        for (int d0 = 0; d0 < cnt; d0 += (WAVE / P) * U) {
                            VT x[U];
#pragma unroll
                            for (int u = 0; u < U; ++u) {                   // distances d0 + k * U + u: a lane's are consecutive
                                const int d = d0 + k * U + u;
                                x[u] = load_agent((const VT*)(gpayA + ((first - (d < cnt ? d : 0)) * nchains + chain) * COLS + pl * VEC));
                            }
                            T part[VEC];
#pragma unroll
                            for (int j = 0; j < VEC; ++j) part[j] = ident;
#pragma unroll
                            for (int u = 0; u < U; ++u) {
                                if (d0 + k * U + u < cnt) {
#pragma unroll
                                    for (int j = 0; j < VEC; ++j) part[j] = op(x[u][j], part[j]);
                                }
                            }
                            for (int delta = P; delta < WAVE; delta <<= 1) {    // lanes further up hold older aggregates
#pragma unroll
                                for (int j = 0; j < VEC; ++j) part[j] = op(__shfl_down(part[j], delta, WAVE), part[j]);
                            }
#pragma unroll
                            for (int j = 0; j < VEC; ++j) acc[j] = op(part[j], acc[j]);     // complete in the lanes below P
                        }
                    } else
                    for (int d0 = 0; d0 < cnt; d0 += 4) {               // four aggregates a round trip
                        VT x[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u)
                            if (d0 + u < cnt) x[u] = load_agent((const VT*)(gpayA + ((first - d0 - u) * nchains + chain) * COLS + lane * VEC));
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            if (d0 + u < cnt) {
#pragma unroll
                                for (int j = 0; j < VEC; ++j) acc[j] = op(x[u][j], acc[j]);
                            }
                        }
                    }
                    if (np >= 0) {
                        if (np >= rem) {                                // ran off the first group: nothing but init in front
#pragma unroll
                            for (int j = 0; j < VEC; ++j) base[j] = op(init, acc[j]);
                        } else {
                            const VT x = load_agent((const VT*)(gpayP + ((first - np) * nchains + chain) * COLS + lane * VEC));
#pragma unroll
                            for (int j = 0; j < VEC; ++j) base[j] = op(x[j], acc[j]);   // a published prefix contains init
                        }
                        break;
                    }
                    first -= WAVE;
                    rem -= WAVE;
                    continue;
                }
                if (wait_give_up(wc, rounds)) break; // `base` is then meaningless
            }
            VT t;
#pragma unroll
            for (int j = 0; j < VEC; ++j) t[j] = base[j];
            store_agent((VT*)(gpayP + ((grp - 1) * nchains + chain) * COLS + lane * VEC), t);
            publish_barrier();
            if (lane == 0) __hip_atomic_store(&gflag[(grp - 1) * nchains + chain], (uint64_t)tagP << 32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    } else {
        // totals of the predecessors inside the group, and the group's base from its leader.  A tile that is not
        // the last of its group needs both before it can go on, so it polls the flags of both together and then has
        // all payloads in flight at once: two round trips instead of four.  The last tile of a group first owes
        // its successors the group aggregate, which needs the predecessors only.
        T local[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) local[j] = ident;
        const bool owes_group = r == ROWS_GROUP - 1 && has_reader;
        const bool with_base = grp > 0 && !owes_group;          // lane 63 polls the leader's flag in the same rounds
        for (;;) {
            uint32_t ok = 1;
            if (lane < r) {
                const uint32_t tag = (uint32_t)(__hip_atomic_load(&desc[(slice - 1 - lane) * nchains + chain], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 32);
                ok = tag == tagA ? 1u : 0u;
            } else if (with_base && lane == WAVE - 1) {
                ok = (uint32_t)(__hip_atomic_load(&gflag[(grp - 1) * nchains + chain], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 32) == tagP ? 1u : 0u;
            }
            if (__ballot(ok == 0u) == 0ull) break;
            if (wait_give_up(wc, rounds)) break;
        }
        VT gbase;
#pragma unroll
        for (int j = 0; j < VEC; ++j) gbase[j] = init;
        {
            VT x[ROWS_GROUP - 1];
#pragma unroll
            for (int d = 0; d < ROWS_GROUP - 1; ++d)
                if (d < r) x[d] = load_agent((const VT*)(payload + ((slice - 1 - d) * nchains + chain) * COLS + lane * VEC));
            if (with_base) gbase = load_agent((const VT*)(gpayP + ((grp - 1) * nchains + chain) * COLS + lane * VEC));
#pragma unroll
            for (int d = 0; d < ROWS_GROUP - 1; ++d) {
                if (d < r) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) local[j] = op(x[d][j], local[j]);
                }
            }
        }
        if (owes_group) {                            // aggregate of the whole group, as soon as it is known
            VT t;
#pragma unroll
            for (int j = 0; j < VEC; ++j) t[j] = op(local[j], tot[j]);
            store_agent((VT*)(gpayA + (grp * nchains + chain) * COLS + lane * VEC), t);
            publish_barrier();
            if (lane == 0) __hip_atomic_store(&gflag[grp * nchains + chain], (uint64_t)tagA << 32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (grp > 0) {                           // then the group's base, from its leader
                for (;;) {
                    uint32_t st = 0;
                    if (lane == 0) st = (uint32_t)(__hip_atomic_load(&gflag[(grp - 1) * nchains + chain], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 32) == tagP ? 1u : 0u;
                    if (__builtin_amdgcn_readfirstlane((int)st) != 0) break;
                    if (wait_give_up(wc, rounds)) break;
                }
                gbase = load_agent((const VT*)(gpayP + ((grp - 1) * nchains + chain) * COLS + lane * VEC));
            }
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) base[j] = op(gbase[j], local[j]);      // a published prefix contains init
    }
}

// NW waves hold rows; one more wave holds none and does the publishing and the look-back.  The registers a kernel
// needs are the maximum over its branches, so the row data (32 registers) and the look-back's working set no longer
// add up: 64 registers suffice and two workgroups share a compute unit (with wave 0 doing both, 25 registers spilled).
template <typename In, typename T, typename Out, typename Op, int NW, int R>
__global__ __launch_bounds__((NW + 1) * WAVE, 8) void scan_rows_ordered_kernel(const In* __restrict__ in, Out* __restrict__ out, ScanGeom g, T init,
                                                                               int inclusive, Op op, int64_t strips, int64_t nchains,
                                                                               int64_t nslices, T* payload, unsigned long long* counter,
                                                                               uint32_t* tickets, int ticket_group, uint64_t* desc,
                                                                               int64_t desc_capacity, WaitCtl wc, int dynamic_ids) {
    constexpr int VEC = 16 / sizeof(T);
    constexpr int COLS = WAVE * VEC;
    typedef typename VecOf<T, VEC>::type VT;
    typedef typename VecOf<In, VEC>::type VI;
    __shared__ T lds[NW][COLS];
    __shared__ T lds_base[COLS];
    const T ident = Op::template identity<T>();
    const int tid = threadIdx.x, wave = tid / WAVE, lane = lane_id();
    const int64_t ntiles = gridDim.x;
    const OrderedId id = ordered_tile_id(counter, dynamic_ids, wave == NW || wave == 0);    // the look-back's wave, and thread 0 at the exit
    const int64_t tile = id.tile;
    const int64_t slice = tile / nchains, chain = tile - slice * nchains;
    const uint32_t epoch = id.epoch;
    wc.stamp = epoch;
    if (wave == NW) {
        __syncthreads();                                 // the row waves have written their column totals
        T tot[VEC], base[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            tot[j] = ident;
#pragma unroll
            for (int w = 0; w < NW; ++w) tot[j] = op(tot[j], lds[w][lane * VEC + j]);
        }
        rows_lookback<T, Op, VEC>(tot, base, init, op, epoch, tile, slice, chain, nchains, nslices, ntiles, payload, desc, wc, lane);
#pragma unroll
        for (int j = 0; j < VEC; ++j) lds_base[lane * VEC + j] = base[j];
        __syncthreads();
    } else {
        const int64_t o = chain / strips, strip = chain - o * strips;
        // rows that are no whole number of vectors: the last vector starts VEC elements before the row's end (see
        // scan_strided_kernel); payloads are per lane slot, the same columns in every tile of the strip
        constexpr bool ANY_ALIGN = sizeof(In) >= 4 && OutElemVectors<Out, T>::value;
        const int64_t nominal = strip * COLS + (int64_t)lane * VEC;
        const bool live = nominal < g.inner;
        const int64_t col0 = (ANY_ALIGN && live && nominal + VEC > g.inner) ? g.inner - VEC : nominal;
        // wave-uniform row addresses + a 32-bit offset per lane (the rows of a wave are the same for all its lanes)
        const int64_t row0 = slice * (NW * R) + (int64_t)__builtin_amdgcn_readfirstlane(wave) * R;
        const int64_t shift = strip * COLS >= VEC ? strip * COLS - VEC : 0;     // the first lane of a strip may reach back VEC columns
        const int64_t wave_e0 = o * g.inner * g.mid + row0 * g.inner + shift;
        const unsigned loff = (unsigned)(col0 - shift);
        const int64_t left = g.mid - row0;
        const int rows = left >= R ? R : (left > 0 ? (int)left : 0);            // rows of this wave inside the array
        VT v[R];
        // (The compiler waits for the second of these loads before it issues the other six, each being under a condition
        // of its own.  Issuing all eight back to back, with clamped addresses instead of conditions, measured slower
        // (4096 x 16384 Float32 105 -> 111 us, 16384 x 4096 99 -> 103 us), and so did a wait after every load (114 us),
        // every second (108) or every fourth (106).)
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (live && r < rows) {
                VI x;
                if constexpr (ANY_ALIGN) x = load_nt_elems<In, VEC>(in + wave_e0 + r * g.inner + loff);
                else x = load_nt((const VI*)(in + wave_e0 + r * g.inner + loff));
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[r][j] = (T)x[j];
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[r][j] = ident;
            }
        }
#pragma unroll
        for (int r = 1; r < R; ++r)
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[r][j] = op(v[r - 1][j], v[r][j]);
#pragma unroll
        for (int j = 0; j < VEC; ++j) lds[wave][lane * VEC + j] = v[R - 1][j];
        __syncthreads();
        T pre[VEC];                                          // the rows of the tile above this wave's
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            pre[j] = ident;
            for (int w = 0; w < wave; ++w) pre[j] = op(pre[j], lds[w][lane * VEC + j]);
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < VEC; ++j) pre[j] = op(lds_base[lane * VEC + j], pre[j]);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (live && r < rows) {
                VT o4;
#pragma unroll
                for (int j = 0; j < VEC; ++j) o4[j] = inclusive ? op(pre[j], v[r][j]) : (r == 0 ? pre[j] : op(pre[j], v[r > 0 ? r - 1 : 0][j]));
                if constexpr (ANY_ALIGN) out_store_elems<Out, T, VEC>(out + wave_e0 + r * g.inner + loff, o4);
                else out_store_nt<Out, T, VEC>(out + wave_e0 + r * g.inner + loff, o4);
            }
        }
    }
    ordered_finish(epoch, ntiles + (nslices + ROWS_GROUP - 1) / ROWS_GROUP * nchains, counter, tickets, ticket_group, desc, desc_capacity);
}

// ---- VEC <= inner <= 32 * VEC, long lines: several rows per load instruction, single pass ----------------------------
// scan_rows_ordered_kernel leaves lanes idle when a row is shorter than its 64 vectors (a row of 64 Float32: 16 of 64
// lanes).  Here P = ceil(inner / VEC) lanes hold a row and a wave's load instruction takes Q = 64 / P consecutive rows --
// a wave covers R * Q consecutive rows, contiguous memory.  Lane group q (lanes q * P .. q * P + P - 1) holds the R
// consecutive rows q * R .. q * R + R - 1 in its registers, lane p of it their p-th vector (the last vector of a row
// that is no whole number of vectors starts VEC elements before the row's end, as in scan_strided_kernel), and scans
// them downwards; one scan of the groups' totals across the lanes (log2 Q steps) joins the groups.  (With the Q rows of a
// load instruction consecutive instead, every register row needs such a scan across the lanes: 64 x 65536 x 16 Float32
// 244 us, of which 100 us for the cross-lane moves.)  The rest is scan_rows_ordered_kernel with a tile of NW * R * Q rows
// and one chain per outer index.  `in` may be `out`: the columns that two lanes hold twice belong to lanes of the same
// load instruction, which is complete before the wave's first store.
template <typename In, typename T, typename Out, typename Op, int NW, int R>
__global__ __launch_bounds__((NW + 1) * WAVE, 8) void scan_rows_packed_kernel(const In* in, Out* out, ScanGeom g, T init, int inclusive, Op op,
                                                                              int P, int64_t nchains, int64_t nslices, T* payload,
                                                                              unsigned long long* counter, uint32_t* tickets, int ticket_group,
                                                                              uint64_t* desc, int64_t desc_capacity, WaitCtl wc, int dynamic_ids) {
    constexpr int VEC = 16 / sizeof(T);
    constexpr int COLS = WAVE * VEC;
    typedef typename VecOf<T, VEC>::type VT;
    typedef typename VecOf<In, VEC>::type VI;
    __shared__ T lds[NW][COLS];
    __shared__ T lds_base[COLS];
    const T ident = Op::template identity<T>();
    const int tid = threadIdx.x, wave = tid / WAVE, lane = lane_id();
    const int64_t ntiles = gridDim.x;
    const OrderedId id = ordered_tile_id(counter, dynamic_ids, wave == NW || wave == 0);    // the look-back's wave, and thread 0 at the exit
    const int64_t tile = id.tile;
    const int64_t slice = tile / nchains, chain = tile - slice * nchains;
    const uint32_t epoch = id.epoch;
    wc.stamp = epoch;
    if (wave == NW) {
        __syncthreads();                                 // the row waves have written their column totals
        T tot[VEC], base[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) tot[j] = ident;
#pragma unroll 5                                         // (all 15 rows in flight at once: 60 registers for 8-byte values)
        for (int w = 0; w < NW; ++w) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) tot[j] = op(tot[j], lds[w][lane * VEC + j]);
        }
        int P2 = 1;                                      // the look-back folds aggregates over power-of-two lane groups
        while (P2 < P) P2 <<= 1;
        rows_lookback<T, Op, VEC, true>(tot, base, init, op, epoch, tile, slice, chain, nchains, nslices, ntiles, payload, desc, wc, lane, P2);
#pragma unroll
        for (int j = 0; j < VEC; ++j) lds_base[lane * VEC + j] = base[j];
        __syncthreads();
    } else {
        const int Q = WAVE / P;
        const int q = lane / P, p = lane - q * P;
        const bool lane_live = q < Q;                     // 64 - P * Q lanes hold nothing
        const int inner = (int)g.inner;
        const int nominal = p * VEC;                      // < inner: P = ceil(inner / VEC)
        const int col0 = nominal + VEC > inner ? inner - VEC : nominal;
        // wave-uniform base + a 32-bit offset per lane: eight 64-bit addresses kept from the loads to the stores would not
        // fit the 64 registers this kernel is compiled for
        const int64_t wave_row0 = (slice * NW + __builtin_amdgcn_readfirstlane(wave)) * (int64_t)(R * Q);
        const int64_t wave_e0 = chain * g.inner * g.mid + wave_row0 * g.inner;
        const int64_t left = g.mid - wave_row0;
        const int rows = left >= R * Q ? R * Q : (left > 0 ? (int)left : 0);      // rows of this wave inside the array
        const int lrow0 = q * R;                          // first row of the lane group, inside the wave's rows
        const unsigned off0 = (unsigned)(lrow0 * inner + col0);
        VT v[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (lane_live && lrow0 + r < rows) {
                const VI x = load_nt_elems<In, VEC>(in + wave_e0 + (off0 + (unsigned)(r * inner)));
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[r][j] = (T)x[j];
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[r][j] = ident;
            }
        }
#pragma unroll
        for (int r = 1; r < R; ++r)
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[r][j] = op(v[r - 1][j], v[r][j]);
        T incl[VEC], excl[VEC];                           // the totals of the lane groups, scanned across the groups
#pragma unroll
        for (int j = 0; j < VEC; ++j) incl[j] = v[R - 1][j];
        for (int delta = P; delta < WAVE; delta <<= 1) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const T y = __shfl_up(incl[j], delta, WAVE);
                if (lane >= delta) incl[j] = op(y, incl[j]);
            }
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            const T up = __shfl_up(incl[j], P, WAVE), all = __shfl(incl[j], (Q - 1) * P + p, WAVE);
            excl[j] = q == 0 ? ident : up;
            lds[wave][lane * VEC + j] = q == 0 ? all : ident;
        }
        __syncthreads();
        T pre[VEC];                                       // the rows of the tile above this wave's
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            pre[j] = ident;
            for (int w = 0; w < wave; ++w) pre[j] = op(pre[j], lds[w][p * VEC + j]);
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < VEC; ++j) pre[j] = op(op(lds_base[p * VEC + j], pre[j]), excl[j]);
        if (!inclusive) {                                 // every row takes the value of the row above it
#pragma unroll
            for (int r = R - 1; r > 0; --r) v[r] = v[r - 1];
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[0][j] = ident;
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (lane_live && lrow0 + r < rows) {
                VT o4;
#pragma unroll
                for (int j = 0; j < VEC; ++j) o4[j] = op(pre[j], v[r][j]);
                out_store_elems<Out, T, VEC>(out + wave_e0 + (off0 + (unsigned)(r * inner)), o4);
            }
        }
    }
    ordered_finish(epoch, ntiles + (nslices + ROWS_GROUP - 1) / ROWS_GROUP * nchains, counter, tickets, ticket_group, desc, desc_capacity);
}

// ---- host side ---------------------------------------------------------------------------------------
template <typename T, int K> struct ScanTile {     // geometry of the tile kernels: 256 threads x K x 16 bytes of output
    static constexpr int VEC = 16 / sizeof(T);
    static constexpr int TILE = 4 * WAVE * VEC * K;
};

int tune_scan_backoff();        // rk_api.hip
int tune_scan_waves();          // rk_api.hip: 0 = choose by line length, else 4, 8 or 16 waves per workgroup
// Waves per workgroup of the single-pass scan of lines of `mid` values of `esz` (>= 4) bytes; a tile is 8 16-byte vectors
// a lane.  Shared with rk_workspace_bytes, which sizes the descriptors for the tiles chosen here.
inline int scan_tile_waves(int64_t mid, size_t esz) {
    if (tune_scan_waves() != 0) return tune_scan_waves();
    const int64_t tile4 = (int64_t)4 * WAVE * (16 / (int64_t)esz) * 8;
    const int64_t tile16 = tile4 * 4, cover16 = (mid + tile16 - 1) / tile16 * tile16;
    return cover16 * 10 <= mid * 11 ? 16 : (mid * (int64_t)esz > ((int64_t)32 << 10) ? 8 : 4);
}
int tune_scan_stagger_ticks();  // rk_api.hip: start-up stagger of the ordered scan in 10 ns ticks across the first resident round
long long wait_budget();        // rk_api.hip: poll rounds a bounded wait may spend (rk_set_wait_budget)
inline WaitAlone wait_alone(WsHeader* hdr) { const long long b = wait_budget(); return WaitAlone{b < WAIT_PATIENCE ? b : WAIT_PATIENCE, &hdr->alone}; }
inline WaitCtl wait_ctl(WsHeader* hdr) { return WaitCtl{&hdr->wait_failed, wait_budget(), tune_scan_backoff(), 0u}; }   // stamp: the kernel's epoch
int tune_scan_blocks_per_cu();  // rk_api.hip
int tune_scan_rows_ordered();    // rk_api.hip: 0 = scans across rows always take the three-pass path
int tune_scan_rows_packed();     // rk_api.hip: 0 = short rows never take the single-pass kernel with several rows per load
int tune_scan_dynamic_ids();     // rk_api.hip: 1 = tile ids from a counter (scan_chain_kernel) instead of launch order
int tune_scan_ordered_unaligned();   // rk_api.hip: 0 = lines at odd addresses take the counter-fed scan_chain_kernel
int tune_scan_tiles_waves();     // rk_api.hip: 0 = the tile-a-line scan always runs four waves a workgroup
int tune_scan_ordered8();        // rk_api.hip: 0 = 8-byte values take the counter-fed scan_chain_kernel
int tune_scan_packed();          // rk_api.hip: 0 = 1- and 2-byte integers never take the packed tiles of the single-pass scan
int tune_scan_slice_blocks_per_cu();  // rk_api.hip: workgroups per compute unit the sliced scan across rows aims for

struct ScanArgs {
    int op;
    const void* in; void* out;
    int ndim; const int64_t* shape; int dim; int inclusive;
    const void* init;
    void* ws; size_t ws_bytes; hipStream_t stream;
};

// Scan along `mid` with lanes along `inner` (inner >= 64).  With enough strips one workgroup per strip walks all
// of `mid` (8 bytes per element).  Otherwise `mid` is cut into slices: totals per slice, an exclusive scan of
// the totals seeded with init (in place in `scratch`; by this function again when there are many slices), then
// the slices scan independently from their carried-in prefix: 12 bytes per element, but the whole device works.
// Short slices are deliberate: workgroups that are resident together then cover a compact range of rows, which
// the memory system serves faster than many rows far apart (measured with power-of-two row strides).
template <typename In, typename T, typename Out, typename Op>
inline int32_t scan_across_rows(const In* in, Out* out, const ScanGeom& g, T init, int inclusive, Op op, bool aligned, char* scratch,
                                size_t scratch_bytes, hipStream_t stream, const Workspace* ws = nullptr) {
    constexpr int VEC = 16 / sizeof(T);
    // 4- and 8-byte elements: vectors at any element-aligned address, rows of any length (>= 64 here)
    // (in place, a row's last vector would re-read columns that the lane before -- possibly of another workgroup -- has
    // already overwritten with results: whole-vector rows only)
    const bool in_place = (const void*)in == (const void*)out;
    const bool vec = (sizeof(In) >= 4 && sizeof(T) >= 4 && !(in_place && g.inner % VEC != 0))
                         ? (is_aligned(in, sizeof(In)) && is_aligned(out, sizeof(Out)) && g.inner >= VEC)
                         : (aligned && g.inner % VEC == 0);
    const int cols = WAVE * (vec ? VEC : 1);
    const int64_t strips = (g.inner + cols - 1) / cols;
    if (strips * g.outer > 0x7fffffff) return RK_ERR_TOO_LARGE;
    const int64_t pitch = strips * cols;
    const int64_t cus = device_info().cus;
    {
        // single pass over tiles of 150 rows (7 waves of rows: 134 us against 109 for the 4096 x 16384 matrix; 15 waves of 8
        // rows 104 us, of 10 rows -- with the row addresses wave-uniform, which freed the registers -- 100, of 12 rows 105);
        // the payloads of all tiles and groups must fit the partials area.  8-byte values too: 2048 x 16384 Float64 103 us against 139
        // for the three passes, 4096 x 4096 Int64 54 against 70.
        constexpr int NW = 15, R = sizeof(In) >= 4 ? 10 : 8;     // 15 waves of rows + 1 for the look-back (Bool -> Int64 with ten rows: 20 registers spilled)
        const int64_t nchains = strips * g.outer, nslices = (g.mid + NW * R - 1) / (NW * R), ntiles = nchains * nslices;
        const int64_t ngroups = (nslices + ROWS_GROUP - 1) / ROWS_GROUP * nchains;
        if (vec && ws != nullptr && tune_scan_rows_ordered() != 0 && nchains < cus * 4 && nslices >= 4 &&
            (size_t)((ntiles + 2 * ngroups) * cols) * sizeof(T) <= scratch_bytes && (size_t)(ntiles + ngroups) * sizeof(uint64_t) <= ws->desc_bytes) {
            scan_rows_ordered_kernel<In, T, Out, Op, NW, R><<<(unsigned)ntiles, (NW + 1) * WAVE, 0, stream>>>(
                in, out, g, init, inclusive, op, strips, nchains, nslices, (T*)scratch, (unsigned long long*)&ws->hdr->scan_counter,
                ws->tickets, ordered_ticket_group(ntiles), ws->desc, (int64_t)(ws->desc_bytes / sizeof(uint64_t)), wait_ctl(ws->hdr),
                ordered_dynamic_ids(ntiles, (NW + 1) * WAVE, rows_chains_stay_on_their_xcd(nchains)));
            RK_LAUNCH_CHECK();
            return RK_SUCCESS;
        }
    }
    int64_t slices = 1;
    if (strips * g.outer < cus * 4) {
        const int64_t want = cus * tune_scan_slice_blocks_per_cu();
        slices = (want + strips * g.outer - 1) / (strips * g.outer);
        const int64_t max_slices = g.mid / 32;                           // at least one register tile of rows per slice
        if (slices > max_slices) slices = max_slices;
        const int64_t fit = (int64_t)(scratch_bytes / 33 * 32 / sizeof(T)) / (pitch * g.outer);   // leave room for the scan of the totals
        if (slices > fit) slices = fit;
        if (slices > 65535) slices = 65535;
    }
    if (slices <= 1) {
        dim3 grid((unsigned)(strips * g.outer), 1);
        if (vec) scan_strided_kernel<In, T, Out, Op, true, 8><<<grid, 256, 0, stream>>>(in, out, g, init, inclusive, op, g.mid, nullptr, 0, strips);
        else     scan_strided_kernel<In, T, Out, Op, false, 8><<<grid, 256, 0, stream>>>(in, out, g, init, inclusive, op, g.mid, nullptr, 0, strips);
        RK_LAUNCH_CHECK();
        return RK_SUCCESS;
    }
    int64_t rps = (g.mid + slices - 1) / slices;
    rps = (rps + 31) / 32 * 32;                                          // whole register tiles (4 waves x 8 rows)
    slices = (g.mid + rps - 1) / rps;
    T* totals = (T*)scratch;
    const size_t used = ((size_t)(pitch * slices * g.outer) * sizeof(T) + 255) & ~(size_t)255;
    dim3 grid((unsigned)(strips * g.outer), (unsigned)slices);
    if (vec) scan_strided_totals_kernel<In, T, Op, true, 4><<<grid, 256, 0, stream>>>(in, totals, g, op, rps, pitch, strips);
    else     scan_strided_totals_kernel<In, T, Op, false, 4><<<grid, 256, 0, stream>>>(in, totals, g, op, rps, pitch, strips);
    RK_LAUNCH_CHECK();
    // exclusive scan of the totals along the slice axis, in place, seeded with init: (pitch, slices, outer); the
    // totals are 16-byte aligned and pitch % VEC == 0
    const ScanGeom tg{pitch, slices, g.outer};
    if (slices > 128) {
        const int32_t st = scan_across_rows<T, T, T, Op>(totals, totals, tg, init, 0, op, true, scratch + used,
                                                      used < scratch_bytes ? scratch_bytes - used : 0, stream);
        if (st != RK_SUCCESS) return st;
    } else {
        const int tcols = WAVE * VEC;
        const int64_t tstrips = (pitch + tcols - 1) / tcols;
        dim3 tgrid((unsigned)(tstrips * g.outer), 1);
        scan_strided_kernel<T, T, T, Op, true, 8><<<tgrid, 256, 0, stream>>>(totals, totals, tg, init, 0, op, slices, nullptr, 0, tstrips);
        RK_LAUNCH_CHECK();
    }
    if (vec) scan_strided_kernel<In, T, Out, Op, true, 8><<<grid, 256, 0, stream>>>(in, out, g, init, inclusive, op, rps, totals, pitch, strips);
    else     scan_strided_kernel<In, T, Out, Op, false, 8><<<grid, 256, 0, stream>>>(in, out, g, init, inclusive, op, rps, totals, pitch, strips);
    RK_LAUNCH_CHECK();
    return RK_SUCCESS;
}

// Scan along `mid` for VEC <= inner <= 32 * VEC in one pass (see scan_rows_packed_kernel).  *done stays false when the
// shape or the workspace does not fit: the caller then takes another path.
template <typename In, typename T, typename Out, typename Op>
inline int32_t scan_rows_packed(const In* in, Out* out, const ScanGeom& g, T init, int inclusive, Op op, const Workspace& w, hipStream_t stream,
                                bool* done) {
    *done = false;
    if constexpr (ElemVectors<In, T>::value) {
        constexpr int VEC = 16 / (int)sizeof(T), COLS = WAVE * VEC;
        constexpr int NW = 15, R = 8;              // (ten rows per lane group: 63 x 500_000 Float32 71 -> 79 us)
        // (rows shorter than a 128-byte line: a load instruction then takes Q short pieces R rows apart, and the two-pass
        // tiles through LDS are two to three times faster: 7 x 4_194_304 Float32 265 against 83 us)
        if (g.inner * sizeof(In) < 128 || g.inner * 2 > COLS || !is_aligned(in, sizeof(In)) || !is_aligned(out, sizeof(Out))) return RK_SUCCESS;
        const int P = (int)((g.inner + VEC - 1) / VEC), Q = WAVE / P;
        const int64_t tile_rows = (int64_t)NW * R * Q;
        const int64_t nchains = g.outer, nslices = (g.mid + tile_rows - 1) / tile_rows;
        if (nslices < 4 || nchains >= (int64_t)device_info().cus * 4 || nslices > 0x7fffffff / nchains) return RK_SUCCESS;
        const int64_t ntiles = nchains * nslices;
        const int64_t ngroups = (nslices + ROWS_GROUP - 1) / ROWS_GROUP * nchains;
        if ((size_t)((ntiles + 2 * ngroups) * COLS) * sizeof(T) > WS_PARTIALS_BYTES || (size_t)(ntiles + ngroups) * sizeof(uint64_t) > w.desc_bytes)
            return RK_SUCCESS;
        scan_rows_packed_kernel<In, T, Out, Op, NW, R><<<(unsigned)ntiles, (NW + 1) * WAVE, 0, stream>>>(
            in, out, g, init, inclusive, op, P, nchains, nslices, (T*)w.partials, (unsigned long long*)&w.hdr->scan_counter, w.tickets,
            ordered_ticket_group(ntiles), w.desc, (int64_t)(w.desc_bytes / sizeof(uint64_t)), wait_ctl(w.hdr), ordered_dynamic_ids(ntiles, (NW + 1) * WAVE, rows_chains_stay_on_their_xcd(nchains)));
        RK_LAUNCH_CHECK();
        *done = true;
    }
    return RK_SUCCESS;
}

// Scan along `mid` for 1 < inner < 64 (see scan_narrow_kernel).  Returns false when the tile totals do not fit the
// scratch area: the caller then takes another path.
template <typename In, typename T, typename Out, typename Op>
inline int32_t scan_narrow(const In* in, Out* out, const ScanGeom& g, T init, int inclusive, Op op, char* scratch, size_t scratch_bytes,
                           hipStream_t stream, bool* done) {
    *done = false;
    constexpr int VEC = 16 / (int)sizeof(T);
    int64_t rows_per_tile = NarrowTile<T>::ELEMS / g.inner;
    // tiles that start at whole vectors: rows_per_tile * inner, and the slab of one outer index, multiples of the vector
    const bool vec = is_aligned(in, VEC * sizeof(In)) && is_aligned(out, VEC * sizeof(Out)) && rows_per_tile >= VEC &&
                     (g.outer == 1 || (g.inner * g.mid) % VEC == 0);
    if (vec) rows_per_tile -= rows_per_tile % VEC;
    const int64_t tiles = (g.mid + rows_per_tile - 1) / rows_per_tile;
    if (tiles > 0x7fffffff || g.outer > 65535) return RK_SUCCESS;
    const size_t need = (size_t)(tiles * g.outer * g.inner) * sizeof(T);
    const size_t used = (need + 255) & ~(size_t)255;
    if (scratch == nullptr || used > scratch_bytes) return RK_SUCCESS;
    T* totals = (T*)scratch;
    dim3 grid((unsigned)tiles, (unsigned)g.outer);
    if (vec) scan_narrow_kernel<In, T, Out, Op, true, true><<<grid, 256, 0, stream>>>(in, nullptr, g, inclusive, op, rows_per_tile, totals, init);
    else scan_narrow_kernel<In, T, Out, Op, true, false><<<grid, 256, 0, stream>>>(in, nullptr, g, inclusive, op, rows_per_tile, totals, init);
    RK_LAUNCH_CHECK();
    // exclusive scan of the totals along the tiles, seeded with init: the (inner, tiles, outer) problem again
    const ScanGeom tg{g.inner, tiles, g.outer};
    if (tiles * g.inner <= NarrowTile<T>::ELEMS && tiles > 32) {
        // all tile totals of an outer index fit one tile: one workgroup each scans them in place
        scan_narrow_kernel<T, T, T, Op, false, false><<<dim3(1, (unsigned)g.outer), 256, 0, stream>>>(totals, totals, tg, 0, op, tiles, nullptr, init);
        RK_LAUNCH_CHECK();
    } else {
        bool sub = false;
        if (tiles > 32) {              // a lane per column walking more tiles than this is slower than three small launches
            const int32_t st = scan_narrow<T, T, T, Op>(totals, totals, tg, init, 0, op, scratch + used, scratch_bytes - used, stream, &sub);
            if (st != RK_SUCCESS) return st;
        }
        if (!sub) {
            const int64_t blocks = (g.inner * g.outer + 255) / 256;
            scan_thread_kernel<T, T, T, Op, 256><<<(unsigned)blocks, 256, 0, stream>>>(totals, totals, tg, init, 0, op);
            RK_LAUNCH_CHECK();
        }
    }
    if (vec) scan_narrow_kernel<In, T, Out, Op, false, true><<<grid, 256, 0, stream>>>(in, out, g, inclusive, op, rows_per_tile, totals, init);
    else scan_narrow_kernel<In, T, Out, Op, false, false><<<grid, 256, 0, stream>>>(in, out, g, inclusive, op, rows_per_tile, totals, init);
    RK_LAUNCH_CHECK();
    *done = true;
    return RK_SUCCESS;
}

template <typename In, typename T, typename Out, typename Op>
inline int32_t launch_scan(const ScanArgs& a) {
    const Op op;
    const T init = a.init ? (T)*(const Out*)a.init : Op::template identity<T>();      // `init` has the output's element type
    const In* in = (const In*)a.in;
    Out* out = (Out*)a.out;
    const uint32_t mask = (a.dim >= 1 && a.dim <= a.ndim) ? (1u << (a.dim - 1)) : 0u;
    const Shape3 s = collapse3(a.ndim, a.shape, mask);
    if (s.total == 0) return RK_SUCCESS;
    ScanGeom g{s.inner, s.mid, s.outer};
    constexpr int VEC = 16 / sizeof(T);
    const bool aligned = is_aligned(in, VEC * sizeof(In)) && is_aligned(out, VEC * sizeof(Out));
    const int inclusive = a.inclusive ? 1 : 0;

    {
        // short lines whose inner x mid slabs fit an LDS tile.  Contiguous lines that are whole vectors have their own
        // kernel below (up to 32 vectors) or do as well with a wave each (beyond 64 elements); with 16 .. 63 elements in
        // a row a lane per line reads whole 64-byte pieces and is faster (32 x 32 x 32768 Float32: 44 against 52 us).
        const int64_t slab = s.inner * s.mid;
        const int64_t all_lines = s.inner * s.outer;
        const bool whole_vectors = aligned && s.inner == 1 && s.mid % VEC == 0 && (s.mid / VEC <= 32 || s.mid > 64);
        if (s.mid >= 2 && all_lines >= 1024 && slab <= (int64_t)(16384 / sizeof(T)) && !whole_vectors &&
            (s.inner > 1 ? (s.inner < 16 || s.inner >= 64) : (s.mid >= 3 && s.mid <= SCAN_LDS_LINES_MAX))) {
            int spb = (int)(16384 / sizeof(T)) / (int)slab;
            bool vector = aligned;
            if (vector) {
                int q = VEC;                                                  // VEC / gcd(slab, VEC)
                for (int64_t e = slab; q > 1 && e % 2 == 0; e /= 2) q /= 2;
                if (spb / q > 0) spb -= spb % q;
                else vector = false;
            }
            int lines = spb * (int)s.inner;
            int tl = 0;
            while (tl < 6 && (lines << tl) < 256 && (2 << tl) <= s.mid) ++tl;            // up to a wave per line
            if (tl == 0 && lines > 256) {
                // a lane per line: whole rounds of 256 lines (273 lines of 15 elements are two rounds, the second with
                // 17 busy lanes); slabs per block stay a multiple of what keeps the blocks 16-byte aligned
                int q = 1;
                if (vector) { q = VEC; for (int64_t e = slab; q > 1 && e % 2 == 0; e /= 2) q /= 2; }
                for (int cand = spb; cand * 4 >= spb * 3 && cand > 0; cand -= q) {
                    if ((cand * (int)s.inner) % 256 == 0) { spb = cand; lines = spb * (int)s.inner; break; }
                }
            }
            if ((lines << tl) >= 128) {                                       // else too few lanes would scan
                const int64_t blocks = (s.outer + spb - 1) / spb;
                if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
                if (vector)
                    scan_lds_lines_kernel<In, T, Out, Op, true><<<(unsigned)blocks, 256, 0, a.stream>>>(in, out, (int)s.inner, (int)s.mid, s.outer, spb, tl, init, inclusive, op);
                else
                    scan_lds_lines_kernel<In, T, Out, Op, false><<<(unsigned)blocks, 256, 0, a.stream>>>(in, out, (int)s.inner, (int)s.mid, s.outer, spb, tl, init, inclusive, op);
                RK_LAUNCH_CHECK();
                return RK_SUCCESS;
            }
        }
    }
    if constexpr (ElemVectors<In, T>::value) {
        // (not in place with rows that are no whole vectors: the row's last group re-reads columns of the group before)
        if (s.inner >= 64 && s.mid <= 16 && s.inner * s.outer >= 4096 && is_aligned(in, sizeof(In)) && is_aligned(out, sizeof(Out)) &&
            !((const void*)in == (const void*)out && s.inner % VEC != 0)) {
            const int64_t groups_per_row = (s.inner + VEC - 1) / VEC;
            if (groups_per_row > INT64_MAX / s.outer) return RK_ERR_TOO_LARGE;
            const int64_t ngroups = groups_per_row * s.outer, blocks = (ngroups + 255) / 256;
            if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
            scan_cols_kernel<In, T, Out, Op><<<(unsigned)blocks, 256, 0, a.stream>>>(in, out, g, init, inclusive, op, groups_per_row, ngroups);
            RK_LAUNCH_CHECK();
            return RK_SUCCESS;
        }
    }
    if (s.inner >= 64) {
        Workspace w{};
        char* scratch = nullptr;
        size_t scratch_bytes = 0;
        const bool have_ws = carve_workspace(a.ws, a.ws_bytes, 0, &w);
        if (have_ws && tune_scan_rows_packed() != 0) {      // rows of at most half a strip of columns
            bool done = false;
            const int32_t st = scan_rows_packed<In, T, Out, Op>(in, out, g, init, inclusive, op, w, a.stream, &done);
            if (st != RK_SUCCESS || done) return st;
        }
        if (have_ws) { scratch = (char*)w.partials; scratch_bytes = WS_PARTIALS_BYTES; }
        return scan_across_rows<In, T, Out, Op>(in, out, g, init, inclusive, op, aligned, scratch, scratch_bytes, a.stream, have_ws ? &w : nullptr);
    }
    const int64_t nlines = s.inner * s.outer;
    if (s.inner > 1 && s.mid > 64) {
        // narrow inner, long lines: whole-row tiles through LDS (one lane per line would walk each line alone:
        // 127 ms for accumulate(+, 3 x 1_000_000; dims=2))
        Workspace w{};
        if (carve_workspace(a.ws, a.ws_bytes, 0, &w)) {
            bool done = false;
            if (tune_scan_rows_packed() != 0) {
                const int32_t st = scan_rows_packed<In, T, Out, Op>(in, out, g, init, inclusive, op, w, a.stream, &done);
                if (st != RK_SUCCESS || done) return st;
            }
            const int32_t st = scan_narrow<In, T, Out, Op>(in, out, g, init, inclusive, op, (char*)w.partials, WS_PARTIALS_BYTES, a.stream, &done);
            if (st != RK_SUCCESS || done) return st;
        }
    }
    if (s.inner == 1 && s.mid % VEC == 0 && s.mid / VEC <= 32 && aligned) {
        const int L = (int)(s.mid / VEC);
        const int64_t per_block = (int64_t)4 * 4 * (64 / L);            // waves x steps x lines per wave and step
        const int64_t blocks = (nlines + per_block - 1) / per_block;
        if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
        scan_short_lines_kernel<In, T, Out, Op, 256><<<(unsigned)blocks, 256, 0, a.stream>>>(in, out, L, nlines, init, inclusive, op);
        RK_LAUNCH_CHECK();
        return RK_SUCCESS;
    }
    if (s.inner > 1 || s.mid <= 16) {
        const int64_t blocks = (nlines + 255) / 256;
        if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
        scan_thread_kernel<In, T, Out, Op, 256><<<(unsigned)blocks, 256, 0, a.stream>>>(in, out, g, init, inclusive, op);
        RK_LAUNCH_CHECK();
        return RK_SUCCESS;
    }
    // contiguous lines
    const bool lines_aligned = aligned && (nlines == 1 || s.mid % VEC == 0);
    if (s.mid <= 1024 && nlines >= 64) {
        const int64_t blocks = (nlines + 3) / 4;
        if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
        if (lines_aligned && s.mid % VEC == 0)
            scan_wave_lines_kernel<In, T, Out, Op, true, 256><<<(unsigned)blocks, 256, 0, a.stream>>>(in, out, s.mid, nlines, init, inclusive, op);
        else
            scan_wave_lines_kernel<In, T, Out, Op, false, 256><<<(unsigned)blocks, 256, 0, a.stream>>>(in, out, s.mid, nlines, init, inclusive, op);
        RK_LAUNCH_CHECK();
        return RK_SUCCESS;
    }
    // lines that fit one tile: smallest tile that holds the line
    if (s.mid <= ScanTile<T, 8>::TILE) {
        if (nlines > 0x7fffffff) return RK_ERR_TOO_LARGE;
        const unsigned grid = (unsigned)nlines;
#define RK_SCAN_TILES(KK)                                                                                             \
        do {                                                                                                          \
            if (lines_aligned) scan_tiles_kernel<In, T, Out, Op, true, KK><<<grid, 256, 0, a.stream>>>(in, out, s.mid, init, inclusive, op); \
            else scan_tiles_kernel<In, T, Out, Op, false, KK><<<grid, 256, 0, a.stream>>>(in, out, s.mid, init, inclusive, op);            \
        } while (0)
        // Aligned lines of 4- and 8-byte elements: two 16-byte loads a lane and as many waves as the line needs (4, 8 or
        // 16) instead of four waves with 2, 4 or 8 loads each -- cumsum(B; dims=1) of 4096 x 16384 Float32 85.3 -> 81.3 us,
        // 3000 x 20000 83.8 -> 81.0, 8192 x 8192 90.2 -> 84.0, 6000 x 10000 84.0 -> 80.9 (the other way round, 16 waves on
        // 16 KiB lines and 8 on 32 KiB ones: 89.6 and 91.4).  Narrow elements, whose loads are 4 or 8 bytes a lane, keep
        // the four waves (Float16 4096 x 16384: 42.5 against 45.8 us).  RK_SCAN_TILES_WAVES=0: four waves always.
        if (lines_aligned && sizeof(In) == sizeof(T) && tune_scan_tiles_waves() != 0 && s.mid > ScanTile<T, 2>::TILE) {
            if (s.mid <= ScanTile<T, 4>::TILE) scan_tiles_kernel<In, T, Out, Op, true, 2, 8><<<grid, 8 * WAVE, 0, a.stream>>>(in, out, s.mid, init, inclusive, op);
            else scan_tiles_kernel<In, T, Out, Op, true, 2, 16><<<grid, 16 * WAVE, 0, a.stream>>>(in, out, s.mid, init, inclusive, op);
        } else
        if (s.mid <= ScanTile<T, 2>::TILE) RK_SCAN_TILES(2);
        else if (s.mid <= ScanTile<T, 4>::TILE) RK_SCAN_TILES(4);
        else RK_SCAN_TILES(8);
#undef RK_SCAN_TILES
        RK_LAUNCH_CHECK();
        return RK_SUCCESS;
    }
    // long lines: single pass with look-back; tile = NW waves x 8 vectors, as large as the line length allows
    constexpr int KT = 8;
    const int64_t line_bytes = s.mid * (int64_t)sizeof(T);
    // measured (4-byte elements): on lines of a megabyte and more 16 waves beat 8 and 4 -- fewer, larger tiles mean fewer
    // look-backs (2^26 elements: 92 against 97 us).  Shorter lines leave the last 128 KiB tile of every line partly
    // empty, and a half-idle workgroup of 1024 threads holds half a compute unit: 3000 lines of 20000 Float32 139 us
    // with 16 waves, 85 us with 8; 1300 lines of 50000: 119 against 97; 600 lines of 100000: 88 against 85
    // -- so 16 waves only where their tiles are at least 90 % full (65536 x 1024 Int32, two full tiles a line: 96 against 101 us)
    // 1- and 2-byte integers on lines of whole, 16-byte aligned vectors that fill tiles of 128 KiB: the packed tiles
    constexpr bool CAN_PACK = std::is_integral<In>::value && std::is_same<In, Out>::value && sizeof(In) <= 2 && sizeof(T) == 4;
    constexpr int PVEC = 16 / (int)sizeof(In);
    const bool packed = CAN_PACK && tune_scan_packed() != 0 && tune_scan_dynamic_ids() == 0 && is_aligned(in, 16) && is_aligned(out, 16) &&
                        s.mid % PVEC == 0 && scan_tile_waves(s.mid, sizeof(In)) == 16;
    const int nw = packed ? 16 : scan_tile_waves(s.mid, sizeof(T));
    const int64_t TILE = packed ? (int64_t)16 * WAVE * PVEC * KT : (int64_t)ScanTile<T, KT>::TILE / 4 * nw;
    const int64_t tpl = (s.mid + TILE - 1) / TILE;
    const int64_t ntiles = tpl * nlines;
    if (ntiles > 0x3fffffff) return RK_ERR_TOO_LARGE;
    Workspace w{};
    const int64_t gpl = (tpl + WAVE - 1) / WAVE, ngroups = gpl * nlines;
    // Unaligned lines do not fit two workgroups a compute unit; with one, the persistent counter-fed kernel is the
    // faster of the two.  8-byte values take the launch-order kernel since their tile scan fits its 64 registers
    // (RK_SCAN_ORDERED8=0: the counter-fed one; cumsum of Int64[2^25] 99.5 -> 88 us, Float64[2^26] 192 -> 173,
    // Bool -> Int64 at 2^26 122 -> 101)
    constexpr bool ORDERED8 = sizeof(T) == 8;
    // lines at odd addresses (or of a length that is no whole number of vectors): the same kernel with 16-byte accesses
    // at element-aligned addresses, where the element types allow them
    constexpr bool ORDERED_ELEMS = ElemVectors<In, T>::value && OutElemVectors<Out, T>::value;
    const bool ordered_unaligned = ORDERED_ELEMS && tune_scan_ordered_unaligned() != 0;
    const bool dynamic_ids = tune_scan_dynamic_ids() != 0 || (sizeof(T) > 4 && !(ORDERED8 && tune_scan_ordered8() != 0)) ||
                             (!lines_aligned && !ordered_unaligned);
    const size_t need = dynamic_ids ? (size_t)(ntiles + ngroups) * Words<T>::N * sizeof(uint64_t)
                                    : ((size_t)ntiles * Words<T>::N + (size_t)ngroups * GROUP_DESC_STRIDE) * sizeof(uint64_t);
    if (!carve_workspace(a.ws, a.ws_bytes, need, &w)) return RK_ERR_WORKSPACE;
    const int64_t cap = (int64_t)(w.desc_bytes / sizeof(uint64_t));
    unsigned long long* counter = (unsigned long long*)&w.hdr->scan_counter;
    const WaitCtl wc = wait_ctl(w.hdr);
    if constexpr (sizeof(T) <= 4 || ORDERED8) {
        if (!dynamic_ids) {
#define RK_SCAN_ORDERED_V(VECF, NWW)                                                                                  \
            scan_ordered_kernel<In, T, Out, Op, VECF, KT, NWW><<<(unsigned)ntiles, NWW * WAVE, 0, a.stream>>>(               \
                in, out, s.mid, tpl, ntiles, init, inclusive, op, counter, w.tickets, ordered_ticket_group(ntiles), w.desc, gpl, ngroups, cap, wc, wait_alone(w.hdr), stagger_ticks, stagger_tiles, dyn)
#define RK_SCAN_ORDERED(NWW)                                                                                          \
            do {                                                                                                      \
                if constexpr (ORDERED_ELEMS) { if (lines_aligned) RK_SCAN_ORDERED_V(true, NWW); else RK_SCAN_ORDERED_V(false, NWW); } \
                else RK_SCAN_ORDERED_V(true, NWW);                                                                    \
            } while (0)
            // staggered start of the first resident round (two workgroups of 16 waves a compute unit), where more rounds
            // follow: 5 us across the round measured best (2^26 Int32: 0 / 2 / 4 / 6 / 8 / 12 / 16 us -> 91.8 / 90.3 / 89.7 /
            // 89.9 / 90.1 / 90.9 / 92.0 us; 2^27: 177.9 -> 174.0 us; half the round late by a fixed time gained nothing)
            const int64_t resident = ordered_resident(nw * WAVE);
            // (narrow elements: half the bytes a tile, half the stagger -- Int16[2^26]: 0 / 1 / 2 / 3 / 4 / 5 / 7 us -> 53.0 / 51.9 / 51.6 /
            // 51.6 / 51.7 / 52.7 / 53.2 us)
            const int stagger_tiles = (nw == 16 && ntiles >= 2 * resident) ? (int)resident : 0;
            const int stagger_ticks = packed ? tune_scan_stagger_ticks() : tune_scan_stagger_ticks() * (int)(sizeof(In) + sizeof(Out)) / (int)(2 * sizeof(T));
            const int dyn = ordered_dynamic_ids(ntiles, nw * WAVE, true);
            if constexpr (CAN_PACK) {
                if (packed) {
                    scan_ordered_kernel<In, T, Out, Op, true, KT, 16, true><<<(unsigned)ntiles, 16 * WAVE, 0, a.stream>>>(
                        in, out, s.mid, tpl, ntiles, init, inclusive, op, counter, w.tickets, ordered_ticket_group(ntiles), w.desc, gpl, ngroups, cap, wc, wait_alone(w.hdr), stagger_ticks, stagger_tiles, dyn);
                    RK_LAUNCH_CHECK();
                    return RK_SUCCESS;
                }
            }
            if (nw == 16) RK_SCAN_ORDERED(16); else if (nw == 8) RK_SCAN_ORDERED(8); else RK_SCAN_ORDERED(4);
#undef RK_SCAN_ORDERED
#undef RK_SCAN_ORDERED_V
            RK_LAUNCH_CHECK();
            return RK_SUCCESS;
        }
    }
    int64_t grid = (int64_t)device_info().cus * tune_scan_blocks_per_cu() * 4 / nw;
    if (grid > ntiles) grid = ntiles;
    if (grid < 1) grid = 1;
#define RK_SCAN_CHAIN(VECF, NWW)                                                                                      \
    scan_chain_kernel<In, T, Out, Op, VECF, KT, NWW><<<(unsigned)grid, NWW * WAVE, 0, a.stream>>>(                          \
        in, out, s.mid, tpl, ntiles, init, inclusive, op, counter, w.desc, gpl, ngroups, cap, wc)
    if (lines_aligned) {
        if (nw == 16) RK_SCAN_CHAIN(true, 16); else if (nw == 8) RK_SCAN_CHAIN(true, 8); else RK_SCAN_CHAIN(true, 4);
    } else {
        if (nw == 16) RK_SCAN_CHAIN(false, 16); else if (nw == 8) RK_SCAN_CHAIN(false, 8); else RK_SCAN_CHAIN(false, 4);
    }
#undef RK_SCAN_CHAIN
    RK_LAUNCH_CHECK();
    return RK_SUCCESS;
}

template <typename In, typename T, typename Out = T>
inline int32_t scan_typed(const ScanArgs& a) {
    switch (a.op) {
        case RK_OP_ADD: return launch_scan<In, T, Out, OpAdd>(a);
        case RK_OP_MUL: return launch_scan<In, T, Out, OpMul>(a);
        case RK_OP_MAX: return launch_scan<In, T, Out, OpMax>(a);
        case RK_OP_MIN: return launch_scan<In, T, Out, OpMin>(a);
        default: break;
    }
    // the bitwise operators: integer element types scanned into their own type
    if constexpr (std::is_integral<T>::value && std::is_same<In, Out>::value) {
        switch (a.op) {
            case RK_OP_AND: return launch_scan<In, T, Out, OpAnd>(a);
            case RK_OP_OR:  return launch_scan<In, T, Out, OpOr>(a);
            case RK_OP_XOR: return launch_scan<In, T, Out, OpXor>(a);
            default: break;
        }
    }
    return a.op >= RK_OP_AND && a.op <= RK_OP_XOR ? RK_ERR_UNSUPPORTED : RK_ERR_INVALID_ARGUMENT;
}

int32_t scan_f32(const ScanArgs&);
int32_t scan_f64(const ScanArgs&);
int32_t scan_i32(const ScanArgs&);
int32_t scan_i64(const ScanArgs&);
int32_t scan_u8_i64(const ScanArgs&);
int32_t scan_u8_i32(const ScanArgs&);
int32_t scan_u32(const ScanArgs&);
int32_t scan_u64(const ScanArgs&);
int32_t scan_i8(const ScanArgs&);       // the narrow types: scanned in 32 bits, stored narrow
int32_t scan_u8(const ScanArgs&);
int32_t scan_i16(const ScanArgs&);
int32_t scan_u16(const ScanArgs&);
int32_t scan_f16(const ScanArgs&);

}  // namespace rk
