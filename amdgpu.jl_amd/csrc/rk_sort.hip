// sort! / sortperm! of vectors (src/kernels/sorting.jl:1-3, which forwards to AcceleratedKernels' merge sort):
// least-significant-digit radix sort, 8 bits per pass.
//
//   sort_init_kernel     clears the control block (and the tile descriptors of small sorts); no memset: graph-safe
//   sort_pass_kernel     a tile of 4096 keys ranks its keys by digit (wave-level match by ballots, counts in LDS), learns
//                        how many keys of each digit the earlier tiles hold, reorders the tile in LDS and writes runs of
//                        equal digits.  The kernel is bound by its vector instructions (about 75 a key, 32 of them the
//                        match), not by memory.
//   sort_finish_kernel   moves the result into the caller's array when an odd number of passes ran
//
// Up to 256 tiles (RK_SORT_LOOKBACK_TILES; 2^20 keys) the counts of the earlier tiles come from a chained look-back (tiles in
// ticket order publish their 256 counts, one lane per digit walks back), and a pass reads and writes every key once:
//   sort_min_kernel      integers: one read of the keys for the smallest mapped key, which every key is taken relative to
//   sort_hist_kernel     one read of the keys: the 256-bin histogram of every digit at once
//   sort_plan_kernel     exclusive scan of every histogram = first output slot of each digit value; passes whose
//                        digit is the same for all keys are skipped (small-range integers need 1-2 passes);
//                        records which buffer each remaining pass reads
// Beyond that the walk becomes the bottleneck -- a descriptor is 2 KiB per step against 16 KiB of keys per tile, and the
// tiles in flight resolve their prefixes nearly one after the other (2^22 Float32: 388 us against 146 us) -- so large
// sorts count before every pass instead:
//   sort_minmax_kernel   integers only: smallest and largest key in one read; passes above the range are skipped
//   sort_upsweep_kernel  the 256 digit counts of every tile (one more read of the keys, at streaming speed)
//   sort_tilescan_kernel exclusive scan of the counts down the tiles in one launch (chunks of tiles; the workgroup
//                        that finishes last scans the chunk totals and the digit totals)
// and their pass kernel gives each XCD a contiguous eighth of the tiles.
//
// Keys are mapped to unsigned integers that sort like Base.isless (-0.0 < 0.0, NaN last; sortperm makes every NaN the
// canonical one so that they are equal keys, sort! keeps their bit patterns), complemented for rev=true; the mapping is
// applied on the first read and undone on the last write.  The sort is stable, so sortperm keeps equal keys in index
// order (also with rev=true, as Base does).
#include <cstddef>
#include <cstdlib>
#include <type_traits>

#include "rk_common.hpp"
#include "rk_scan_impl.hpp"

namespace rk {

constexpr int SORT_BLOCK = 256;
constexpr int SORT_NW = SORT_BLOCK / WAVE;
constexpr int SORT_MAX_PASSES = 8;

struct SortCtl {                                  // head of the caller's temporary buffer
    uint32_t hist[SORT_MAX_PASSES][256];          // counts, then (sort_plan_kernel) exclusive prefix sums
    uint32_t ticket[SORT_MAX_PASSES];
    uint32_t skip[SORT_MAX_PASSES];
    uint32_t src_is_b[SORT_MAX_PASSES];           // the pass reads buffer B (1) or A (0)
    uint32_t first_pass, last_pass, nexec;
    uint32_t wait_failed;                         // a look-back gave up its bounded wait (WaitCtl); read by rk_sort_status
    unsigned long long inv_min;                   // ~(smallest mapped key), kept as a maximum so that zero is its identity
    unsigned long long key_max;                   // largest mapped key (large integer sorts: range = key_max - smallest)
    uint32_t scan_ticket[SORT_MAX_PASSES];        // sort_tilescan_kernel: workgroups that have stored their chunk totals
};

// ---- key <-> ordered unsigned integer -----------------------------------------------------------------
template <typename T> struct SortKey;
template <> struct SortKey<int16_t> {
    typedef uint16_t U;
    static __device__ __forceinline__ U enc(int16_t v, bool) { return (U)((uint16_t)v ^ 0x8000u); }
    static __device__ __forceinline__ int16_t dec(U u, bool) { return (int16_t)(u ^ 0x8000u); }
};
template <> struct SortKey<int32_t> {
    typedef uint32_t U;
    static __device__ __forceinline__ U enc(int32_t v, bool) { return (U)v ^ 0x80000000u; }
    static __device__ __forceinline__ int32_t dec(U u, bool) { return (int32_t)(u ^ 0x80000000u); }
};
template <> struct SortKey<int64_t> {
    typedef uint64_t U;
    static __device__ __forceinline__ U enc(int64_t v, bool) { return (U)v ^ 0x8000000000000000ull; }
    static __device__ __forceinline__ int64_t dec(U u, bool) { return (int64_t)(u ^ 0x8000000000000000ull); }
};
// Floats: sign-magnitude bits -> unsigned integers in isless order (-0.0 < 0.0), NaN after +Inf.
//   keep == false (sortperm: the keys are not part of the result): every NaN becomes the canonical one, so all NaNs
//                 are equal keys and stay in index order, as isless-equal elements must in a stable sort.
//   keep == true  (sort!): a bijection of the bit patterns, so the sorted array is a permutation of the input, NaN signs
//                 and payloads included.  The plain mapping puts the negative NaNs below -Inf: NLOW of them, keys
//                 0 .. NLOW-1; they are moved above the positive NaNs and everything else shifts down by NLOW.  The
//                 order among NaNs is then by bit pattern, not by index (Base's own float sort moves its NaNs to the
//                 end without keeping their order either).
template <typename U, U NLOW> struct FloatKeyMap {
    static __device__ __forceinline__ U fwd(U std_key) { return std_key < NLOW ? (U)(std_key + (U)(0 - NLOW)) : (U)(std_key - NLOW); }
    static __device__ __forceinline__ U inv(U k) { return k >= (U)(0 - NLOW) ? (U)(k - (U)(0 - NLOW)) : (U)(k + NLOW); }
};
struct half_bits { uint16_t b; };                 // Float16 travels as its bit pattern
template <> struct SortKey<half_bits> {
    typedef uint16_t U;
    typedef FloatKeyMap<uint16_t, 0x03ffu> Map;    // 0xfc01 .. 0xffff are the negative NaNs
    static __device__ __forceinline__ U enc(half_bits v, bool keep) {
        uint16_t b = v.b;
        if (!keep && (b & 0x7fffu) > 0x7c00u) b = 0x7e00u;        // NaN -> canonical, sorts after +Inf
        const U u = (U)((b & 0x8000u) ? ~b : (b ^ 0x8000u));
        return keep ? Map::fwd(u) : u;
    }
    static __device__ __forceinline__ half_bits dec(U k, bool keep) {
        const U u = keep ? Map::inv(k) : k;
        return half_bits{(uint16_t)((u & 0x8000u) ? (u ^ 0x8000u) : ~u)};
    }
};
template <> struct SortKey<float> {
    typedef uint32_t U;
    typedef FloatKeyMap<uint32_t, 0x007fffffu> Map;
    static __device__ __forceinline__ U enc(float v, bool keep) {
        uint32_t b = __builtin_bit_cast(uint32_t, v);
        if (!keep && v != v) b = 0x7fc00000u;
        const U u = (b & 0x80000000u) ? ~b : (b ^ 0x80000000u);
        return keep ? Map::fwd(u) : u;
    }
    static __device__ __forceinline__ float dec(U k, bool keep) {
        const U u = keep ? Map::inv(k) : k;
        return __builtin_bit_cast(float, (u & 0x80000000u) ? (u ^ 0x80000000u) : ~u);
    }
};
template <> struct SortKey<double> {
    typedef uint64_t U;
    typedef FloatKeyMap<uint64_t, 0x000fffffffffffffull> Map;
    static __device__ __forceinline__ U enc(double v, bool keep) {
        uint64_t b = __builtin_bit_cast(uint64_t, v);
        if (!keep && v != v) b = 0x7ff8000000000000ull;
        const U u = (b & 0x8000000000000000ull) ? ~b : (b ^ 0x8000000000000000ull);
        return keep ? Map::fwd(u) : u;
    }
    static __device__ __forceinline__ double dec(U k, bool keep) {
        const U u = keep ? Map::inv(k) : k;
        return __builtin_bit_cast(double, (u & 0x8000000000000000ull) ? (u ^ 0x8000000000000000ull) : ~u);
    }
};

// `rev` here is a set of flags: bit 0 = descending order, bit 1 = keep NaN bit patterns (SORT_KEEP_NAN).
constexpr int SORT_REV = 1, SORT_KEEP_NAN = 2;
// the same mapping on the raw bit pattern: one load path serves the first pass (caller's keys) and the later ones
// and relative to the smallest mapped key of the array: small-range integers (and floats of one binade) then have
// constant high digits, whose passes are skipped
template <typename T> __device__ __forceinline__ typename SortKey<T>::U enc_bits(typename SortKey<T>::U raw, int rev, typename SortKey<T>::U umin) {
    typedef typename SortKey<T>::U U;
    const U u = SortKey<T>::enc(__builtin_bit_cast(T, raw), (rev & SORT_KEEP_NAN) != 0);
    return (U)(((rev & SORT_REV) ? (U)~u : u) - umin);
}
template <typename T> __device__ __forceinline__ T dec_bits(typename SortKey<T>::U k, int rev, typename SortKey<T>::U umin) {
    typedef typename SortKey<T>::U U;
    const U u = (U)(k + umin);
    return SortKey<T>::dec((rev & SORT_REV) ? (U)~u : u, (rev & SORT_KEEP_NAN) != 0);
}

template <typename U> __device__ __forceinline__ uint32_t digit_of(U u, int pass) { return (uint32_t)(u >> (8 * pass)) & 0xffu; }

// Mask of the lanes of `valid` whose digit equals this lane's.  Per bit of the digit: e = all ones where the bit is
// set, m = ballot of the bit; (m ^ e) has a one exactly for the lanes that differ from this lane in that bit.
__device__ __forceinline__ uint64_t match_digit(uint32_t d, uint64_t valid) {
    uint32_t diff_lo = 0, diff_hi = 0;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const uint32_t e = (uint32_t)__builtin_amdgcn_sbfe((int)d, b, 1);
        const uint64_t m = __ballot(e != 0u);
        diff_lo |= (uint32_t)m ^ e;
        diff_hi |= (uint32_t)(m >> 32) ^ e;
    }
    return ~(((uint64_t)diff_hi << 32) | diff_lo) & valid;
}
// The same for the ranking of the pass kernel, which is bound by its vector instructions: four per bit (sign-extended
// bit, compare into a lane mask, and one three-input bit operation same &= ~(m ^ e) for each half of the wave)
// instead of the six the compiler makes of the plain form.  Call with all 64 lanes active.
__device__ __forceinline__ void match_digit_halves(uint32_t d, uint32_t& same_lo, uint32_t& same_hi) {
    same_lo = ~0u;
    same_hi = ~0u;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const uint32_t e = (uint32_t)__builtin_amdgcn_sbfe((int)d, b, 1);
        uint64_t m;
        asm volatile("v_cmp_ne_u32_e64 %0, 0, %1" : "=s"(m) : "v"(e));
        same_lo = __builtin_amdgcn_bitop3_b32(same_lo, (uint32_t)m, e, 0x90);             // a & ~(b ^ c)
        same_hi = __builtin_amdgcn_bitop3_b32(same_hi, (uint32_t)(m >> 32), e, 0x90);
    }
}

// Histogram updates in LDS.  Evenly spread digits go in with one LDS atomic per lane.  When many lanes hold the same
// digit (exponent bytes, the high bytes of small integers) those atomics would queue up on one LDS word, so the
// lanes are matched first and one lane per digit value adds the whole group.  digits_skewed() is the wave-uniform
// test: do at least 8 lanes share the first lane's digit?
__device__ __forceinline__ bool digits_skewed(uint32_t d, bool valid) {
    const uint64_t active = __ballot(valid);
    if (active == 0ull) return false;
    const uint32_t d0 = (uint32_t)__builtin_amdgcn_readlane((int)d, __ffsll((unsigned long long)active) - 1);
    return __popcll(__ballot(valid && d == d0)) >= 8;
}
__device__ __forceinline__ void count_digit(uint32_t* row, uint32_t d, bool valid, bool skewed) {
    if (skewed) {
        const uint64_t active = __ballot(valid);
        if (active == 0ull) return;
        const int first = __ffsll((unsigned long long)active) - 1;
        const uint32_t d0 = (uint32_t)__builtin_amdgcn_readlane((int)d, first);
        if (__ballot(valid && d == d0) == active) {                       // one value in the whole wave
            if (lane_id() == first) atomicAdd(&row[d0], (uint32_t)__popcll(active));
            return;
        }
        const uint64_t peers = match_digit(d, active);
        if (valid && lane_id() == __ffsll((unsigned long long)peers) - 1) atomicAdd(&row[d], (uint32_t)__popcll(peers));
    } else if (valid) atomicAdd(&row[d], 1u);
}

// ---- init: clear control block and descriptors ------------------------------------------------------------
// min_is_zero: the keys are not taken relative to their smallest (floats: the read that finds it saves no pass), so the
// control block starts with ~0 in inv_min, i.e. a smallest mapped key of 0.
__global__ __launch_bounds__(256) void sort_init_kernel(uint64_t* words, int64_t nwords, int min_is_zero) {
    constexpr int64_t INV_MIN_WORD = (int64_t)(offsetof(SortCtl, inv_min) / sizeof(uint64_t));
    static_assert(offsetof(SortCtl, inv_min) % sizeof(uint64_t) == 0, "inv_min is one of the cleared words");
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nwords; i += (int64_t)gridDim.x * 256)
        words[i] = (min_is_zero && i == INV_MIN_WORD) ? ~0ull : 0ull;
}

// The two whole-array reads below take 16-byte vectors from the aligned body [head, head + nvec * VEC) of the keys
// and single elements from the few keys in front of and behind it.
template <typename T, typename F>
__device__ __forceinline__ void for_each_key(const T* __restrict__ keys, int64_t n, int64_t head, int64_t nvec, F&& f) {
    typedef typename SortKey<T>::U U;
    constexpr int VEC = 16 / sizeof(T);
    typedef typename VecOf<U, VEC>::type VU;
    const VU* body = (const VU*)(keys + head);
    constexpr int UNR = 4;                                   // loads in flight per lane
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i + (UNR - 1) * stride < nvec; i += UNR * stride) {
        VU v[UNR];
#pragma unroll
        for (int r = 0; r < UNR; ++r) v[r] = load_nt(body + i + r * stride);
#pragma unroll
        for (int r = 0; r < UNR; ++r) {
            U k[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) k[j] = (U)v[r][j];
            f(k, VEC);
        }
    }
    for (; i < nvec; i += stride) {
        const VU v = load_nt(body + i);
        U k[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) k[j] = (U)v[j];
        f(k, VEC);
    }
    if (blockIdx.x == 0) {
        const int64_t tail0 = head + nvec * VEC, extra = head + (n - tail0);     // at most 2 * (VEC - 1) keys
        for (int64_t i = threadIdx.x; i < extra; i += blockDim.x) {
            const int64_t e = i < head ? i : tail0 + (i - head);
            U k[VEC];
            k[0] = __builtin_bit_cast(U, keys[e]);
            f(k, 1);
        }
    }
}

// ---- smallest mapped key ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void sort_min_kernel(const T* __restrict__ keys, int64_t n, int64_t head, int64_t nvec, int rev,
                                                       SortCtl* ctl) {
    typedef typename SortKey<T>::U U;
    constexpr int VEC = 16 / sizeof(T);
    __shared__ unsigned long long part[SORT_NW];
    unsigned long long inv = 0;                  // max of ~u
    for_each_key<T>(keys, n, head, nvec, [&](const U (&k)[VEC], int cnt) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            if (j < cnt) {
                const unsigned long long x = (unsigned long long)(U)~enc_bits<T>(k[j], rev, (U)0);
                inv = x > inv ? x : inv;
            }
        }
    });
    // one device-wide atomic per workgroup: atomics on one address complete one after the other
    inv = wave_reduce(inv, OpMax());
    if (lane_id() == 0) part[threadIdx.x / WAVE] = inv;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < SORT_NW; ++w) inv = part[w] > inv ? part[w] : inv;
        if (inv != 0ull) atomicMax(&ctl->inv_min, inv);
    }
}

// ---- smallest and largest mapped key (large integer sorts) ------------------------------------------------------------
// Keys are taken relative to the smallest one, so their range tells which digits are zero in every key: the passes of
// those digits are skipped.  One read at streaming speed; the large sorts do without the histogram read below.
constexpr int MINMAX_BLOCK = 1024;      // few, large workgroups: each ends with two device-wide atomics on shared words
template <typename T>
__global__ __launch_bounds__(MINMAX_BLOCK) void sort_minmax_kernel(const T* __restrict__ keys, int64_t n, int64_t head, int64_t nvec, int rev,
                                                                   SortCtl* ctl) {
    typedef typename SortKey<T>::U U;
    constexpr int VEC = 16 / sizeof(T);
    __shared__ U part[2][MINMAX_BLOCK / WAVE];
    U mn = (U)~(U)0, mx = 0;
    for_each_key<T>(keys, n, head, nvec, [&](const U (&k)[VEC], int cnt) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            if (j < cnt) {
                const U u = enc_bits<T>(k[j], rev, (U)0);
                mn = u < mn ? u : mn;
                mx = u > mx ? u : mx;
            }
        }
    });
    mn = wave_reduce(mn, OpMin());
    mx = wave_reduce(mx, OpMax());
    if (lane_id() == 0) { part[0][threadIdx.x / WAVE] = mn; part[1][threadIdx.x / WAVE] = mx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < MINMAX_BLOCK / WAVE; ++w) { mn = part[0][w] < mn ? part[0][w] : mn; mx = part[1][w] > mx ? part[1][w] : mx; }
        const unsigned long long inv = (unsigned long long)(U)~mn;
        if (inv != 0ull) atomicMax(&ctl->inv_min, inv);
        if (mx != 0) atomicMax(&ctl->key_max, (unsigned long long)mx);
    }
}

// ---- all digit histograms in one read -------------------------------------------------------------------------
template <typename T, int PASSES>
__global__ __launch_bounds__(256) void sort_hist_kernel(const T* __restrict__ keys, int64_t n, int64_t head, int64_t nvec, int rev,
                                                        SortCtl* ctl) {
    typedef typename SortKey<T>::U U;
    __shared__ uint32_t h[PASSES][256];
    const U umin = (U)~ctl->inv_min;
    for (int i = threadIdx.x; i < PASSES * 256; i += 256) (&h[0][0])[i] = 0;
    __syncthreads();
    constexpr int VEC = 16 / sizeof(T);
    for_each_key<T>(keys, n, head, nvec, [&](const U (&k)[VEC], int cnt) {
        U u[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) u[j] = enc_bits<T>(k[j], rev, umin);
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const bool skewed = digits_skewed(digit_of(u[0], p), true);       // judged on the first key of the vector
#pragma unroll
            for (int j = 0; j < VEC; ++j) count_digit(h[p], digit_of(u[j], p), j < cnt, skewed);
        }
    });
    __syncthreads();
    for (int i = threadIdx.x; i < PASSES * 256; i += 256) {
        const uint32_t c = (&h[0][0])[i];
        if (c) atomicAdd(&ctl->hist[0][0] + i, c);
    }
}

// ---- plan: scan the histograms, decide which passes run and what they read ---------------------------------------
// one workgroup of 256 threads; lane d owns digit value d.  mode 0: from the histograms of sort_hist_kernel.
// mode 1 (large sorts of integers): from the range of the keys, histograms come later, pass by pass.
// mode 2 (large sorts of floats): every pass runs, keys are not taken relative to the smallest.
__global__ __launch_bounds__(256) void sort_plan_kernel(SortCtl* ctl, int passes, uint32_t n, int first_reads_b, int mode) {
    __shared__ uint32_t wsum[SORT_NW];
    __shared__ int any_full;
    const int d = threadIdx.x, wave = d / WAVE, lane = d % WAVE;
    if (mode == 0) {
        for (int p = 0; p < passes; ++p) {
            const uint32_t c = ctl->hist[p][d];
            if (d == 0) any_full = 0;
            __syncthreads();
            if (c == n) any_full = 1;
            const uint32_t inc = wave_scan_inclusive(c, OpAdd(), 0u);
            if (lane == WAVE - 1) wsum[wave] = inc;
            __syncthreads();
            uint32_t base = 0;
            for (int w = 0; w < wave; ++w) base += wsum[w];
            ctl->hist[p][d] = base + inc - c;
            if (d == 0) ctl->skip[p] = any_full ? 1u : 0u;
            __syncthreads();
        }
    } else if (d == 0) {
        if (mode == 2) ctl->inv_min = ~0ull;                          // smallest key taken as 0
        const unsigned long long umin = ~ctl->inv_min;                 // high bits beyond the key width: ones in both, cancel below
        const unsigned long long range = mode == 2 ? ~0ull : ctl->key_max - (umin & (passes == 8 ? ~0ull : ((1ull << (8 * passes)) - 1ull)));
        for (int p = 0; p < passes; ++p) ctl->skip[p] = (range >> (8 * p)) == 0ull ? 1u : 0u;
    }
    if (d == 0) {
        uint32_t src_b = first_reads_b ? 1u : 0u, nexec = 0, first = 0xffffffffu, last = 0xffffffffu;
        for (int p = 0; p < passes; ++p) {
            if (ctl->skip[p]) continue;
            ctl->src_is_b[p] = src_b;
            src_b ^= 1u;
            if (first == 0xffffffffu) first = (uint32_t)p;
            last = (uint32_t)p;
            ++nexec;
        }
        ctl->first_pass = first;
        ctl->last_pass = last;
        ctl->nexec = nexec;
    }
}

// ---- digit counts of every tile (large sorts) ---------------------------------------------------------------------
// Same tiles as sort_pass_kernel, one per workgroup; the order of the keys inside the tile does not matter here, so
// aligned full tiles are read as 16-byte vectors.  One LDS atomic per key into one of UPS_SUB histograms per wave,
// chosen by the lane: skewed digits (exponent bytes, the high bytes of small integers) then queue up 16 deep on a
// counter instead of 64 deep, and no lane has to find out who else holds its digit.
constexpr int UPS_SUB = 4;

template <typename T, int ITEMS>
__global__ __launch_bounds__(SORT_BLOCK, 8) void sort_upsweep_kernel(const T* __restrict__ orig, const typename SortKey<T>::U* buf_a,
                                                                  const typename SortKey<T>::U* buf_b, uint32_t n, int pass, int rev,
                                                                  const SortCtl* ctl, uint32_t* __restrict__ tile_count) {
    typedef typename SortKey<T>::U U;
    constexpr int TILE = SORT_BLOCK * ITEMS;
    constexpr int VEC = 16 / (int)sizeof(T), NV = ITEMS / VEC;
    typedef typename VecOf<U, VEC>::type VU;
    __shared__ uint32_t cnt[SORT_NW * UPS_SUB][256];
    if (ctl->skip[pass]) return;
    const bool first = (uint32_t)pass == ctl->first_pass;
    const U* in = first ? (const U*)orig : (ctl->src_is_b[pass] != 0u ? buf_b : buf_a);
    const U umin = (U)~ctl->inv_min;
    const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
    for (int i = tid; i < SORT_NW * UPS_SUB * 256; i += SORT_BLOCK) (&cnt[0][0])[i] = 0;
    const uint32_t tile = blockIdx.x;
    const uint32_t e0 = tile * (uint32_t)TILE;
    const uint32_t woff = e0 + (uint32_t)wave * (WAVE * ITEMS) + lane;
    uint32_t* row = cnt[wave * UPS_SUB + (lane & (UPS_SUB - 1))];
    // When many lanes hold the same digit (judged on every fourth key) the two most frequent values -- as seen from the
    // first lane still in play -- are taken out with a ballot each and added by that lane alone; uniform floats have
    // 50% and 37% of their keys in two values of the exponent digit.
    bool skewed = false;
    auto count = [&](uint32_t d, bool valid, int i) {
        if ((i & 3) == 0) skewed = digits_skewed(d, valid);
        if (skewed) {
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const uint64_t active = __ballot(valid);
                if (active != 0ull) {
                    const int head = __ffsll((unsigned long long)active) - 1;
                    const uint32_t d0 = (uint32_t)__builtin_amdgcn_readlane((int)d, head);
                    const uint64_t same = __ballot(valid && d == d0);
                    if (lane == head) atomicAdd(&row[d0], (uint32_t)__popcll(same));
                    valid = valid && d != d0;
                }
            }
        }
        if (valid) atomicAdd(&row[d], 1u);
    };
    // (the two read paths share no variables: merged into one key array they made the compiler shuffle it through
    // private memory)
    if (e0 + (uint32_t)TILE <= n && (((uintptr_t)(in + e0)) & 15) == 0) {
        const VU* vin = (const VU*)(in + e0);
        VU v[NV];
#pragma unroll
        for (int r = 0; r < NV; ++r) v[r] = vin[r * SORT_BLOCK + tid];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < NV; ++r) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                U k = (U)v[r][j];
                if (first) k = enc_bits<T>(k, rev, umin);
                count(digit_of(k, pass), true, r * VEC + j);
            }
        }
    } else {
        U key[ITEMS];
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const uint32_t e = woff + i * WAVE;
            key[i] = (U)0;
            if (e < n) key[i] = in[e];
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const U k = first ? enc_bits<T>(key[i], rev, umin) : key[i];
            count(digit_of(k, pass), woff + i * WAVE < n, i);
        }
    }
    __syncthreads();
    uint32_t c = 0;
#pragma unroll
    for (int w = 0; w < SORT_NW * UPS_SUB; ++w) c += cnt[w][tid];
    tile_count[(uint64_t)tile * 256 + tid] = c;
}

// ---- where every tile's keys go (large sorts) --------------------------------------------------------------------------
// Input: count[tile][digit].  Output, for sort_pass_kernel: count[tile][digit] becomes the number of keys of the digit in
// the earlier tiles of the same chunk of `chunk_rows` tiles; chunk_prefix[chunk][digit] the number in all earlier chunks;
// ctl->hist[pass][digit] the first output slot of the digit (exclusive scan of the digit totals).
// One workgroup of 1024 threads per chunk: 4 groups of rows x 256 digits.  The workgroup that stores its chunk totals
// last (a ticket) scans the totals of all chunks; nobody waits for anybody.  At most 256 chunks.
constexpr int TS_GROUPS = 4, TS_BLOCK = TS_GROUPS * 256, TS_UNROLL = 16, TS_MAX_CHUNKS = 256;

// Rows [first, first + rows) of column d of x (256 words a row), TS_UNROLL loads in flight: their sum; with WRITE,
// out[row][d] = start + the sum of the rows in front.
template <bool WRITE, bool COHERENT>
__device__ __forceinline__ uint32_t ts_rows(const uint32_t* x, uint32_t first, uint32_t rows, uint32_t d, uint32_t start, uint32_t* out) {
    uint32_t run = start;
    for (uint32_t r = 0; r < rows; r += TS_UNROLL) {
        uint32_t v[TS_UNROLL];
#pragma unroll
        for (int j = 0; j < TS_UNROLL; ++j) {
            v[j] = 0;
            if (r + j < rows) {
                const uint32_t* q = x + (uint64_t)(first + r + j) * 256 + d;
                v[j] = COHERENT ? load_agent(q) : *q;
            }
        }
#pragma unroll
        for (int j = 0; j < TS_UNROLL; ++j) {
            if (WRITE && r + j < rows) out[(uint64_t)(first + r + j) * 256 + d] = run;
            run += v[j];
        }
    }
    return run - start;
}

// Exclusive scan down rows [a, b) of column d, for the thread of row group g: out[row][d] = sum of the rows of the
// column in front, over all groups; returns the column total.  Up to MAXR rows a group stay in registers between the
// two steps (one round trip to memory); longer groups are read twice.
template <int MAXR, bool COHERENT>
__device__ __forceinline__ uint32_t ts_scan_groups(const uint32_t* x, uint32_t* out, uint32_t a, uint32_t b, uint32_t d, uint32_t g,
                                                   uint32_t (*gsum)[256]) {
    const uint32_t rows = b - a;
    const bool in_regs = __syncthreads_and(rows <= (uint32_t)MAXR) != 0;
    uint32_t v[MAXR];
    uint32_t mine = 0;
    if (in_regs) {
#pragma unroll
        for (int j = 0; j < MAXR; ++j) {
            v[j] = 0;
            if ((uint32_t)j < rows) {
                const uint32_t* q = x + (uint64_t)(a + j) * 256 + d;
                v[j] = COHERENT ? load_agent(q) : *q;
            }
        }
#pragma unroll
        for (int j = 0; j < MAXR; ++j) mine += v[j];
    } else {
        mine = ts_rows<false, COHERENT>(x, a, rows, d, 0u, nullptr);
    }
    gsum[g][d] = mine;
    __syncthreads();
    uint32_t before = 0, total = 0;
#pragma unroll
    for (int k = 0; k < TS_GROUPS; ++k) {
        const uint32_t s = gsum[k][d];
        if ((uint32_t)k < g) before += s;
        total += s;
    }
    if (in_regs) {
        uint32_t run = before;
#pragma unroll
        for (int j = 0; j < MAXR; ++j) {
            if ((uint32_t)j < rows) out[(uint64_t)(a + j) * 256 + d] = run;
            run += v[j];
        }
    } else {
        ts_rows<true, COHERENT>(x, a, rows, d, before, out);
    }
    return total;
}

__global__ __launch_bounds__(TS_BLOCK) void sort_tilescan_kernel(SortCtl* ctl, int pass, uint32_t* count, uint32_t ntiles, uint32_t chunk_rows,
                                                                 uint32_t* chunk_total, uint32_t* chunk_prefix) {
    __shared__ uint32_t gsum[2][TS_GROUPS][256];
    __shared__ uint32_t wsum[SORT_NW];
    __shared__ uint32_t lds_ticket;
    if (ctl->skip[pass]) return;
    const uint32_t d = threadIdx.x & 255u, g = threadIdx.x >> 8, chunk = blockIdx.x, nchunks = gridDim.x;
    {
        const uint32_t r0 = chunk * chunk_rows, r1 = r0 + chunk_rows < ntiles ? r0 + chunk_rows : ntiles;
        const uint32_t per = (r1 - r0 + TS_GROUPS - 1) / TS_GROUPS;
        const uint32_t a = r0 + g * per < r1 ? r0 + g * per : r1, b = a + per < r1 ? a + per : r1;
        const uint32_t total = ts_scan_groups<16, false>(count, count, a, b, d, g, gsum[0]);
        if (g == 0) store_agent(chunk_total + (uint64_t)chunk * 256 + d, total);
    }
    publish_barrier();                       // this thread's total is visible device-wide ...
    __syncthreads();                         // ... and so is every other thread's of this workgroup
    if (threadIdx.x == 0) lds_ticket = atomicAdd(&ctl->scan_ticket[pass], 1u);
    __syncthreads();
    if (lds_ticket != nchunks - 1u) return;
    // the last one: exclusive scan of the chunk totals down the chunks, then of the digit totals across the digits
    const uint32_t per = (nchunks + TS_GROUPS - 1) / TS_GROUPS;
    const uint32_t a = g * per < nchunks ? g * per : nchunks, b = a + per < nchunks ? a + per : nchunks;
    const uint32_t total = ts_scan_groups<TS_MAX_CHUNKS / TS_GROUPS, true>(chunk_total, chunk_prefix, a, b, d, g, gsum[1]);
    const uint32_t inc = wave_scan_inclusive(total, OpAdd(), 0u);          // the same in all four groups
    if (g == 0 && d % WAVE == WAVE - 1) wsum[d / WAVE] = inc;
    __syncthreads();
    if (g == 0) {
        uint32_t start = inc - total;
        for (uint32_t w = 0; w < d / WAVE; ++w) start += wsum[w];
        ctl->hist[pass][d] = start;
    }
}

// ---- one pass ----------------------------------------------------------------------------------------------------
// Tile = 256 threads x ITEMS keys.  Wave w owns the w-th quarter of the tile; its item i of lane l is key
// i * 64 + l of that quarter (coalesced loads; the order (i, l) is memory order, which the ranking keeps).
// desc[tile][digit]: low half = count, high half = (pass + 1) << 2 | status (1 = count of this tile only,
// 2 = count of this and all earlier tiles); written and read with relaxed device-scope atomics, so the count
// always travels with its tag.
// waves per SIMD the register allocation aims at: the kernel is bound by its vector instructions, and three or four
// waves hide the latencies (measured: 4 against 6 workgroups a CU differ by 4%)
template <typename T, bool PERM, bool COUNTED> constexpr int sort_pass_waves() { return (COUNTED && !PERM && sizeof(T) <= 4) ? 4 : 3; }

template <typename T, int ITEMS, bool PERM, bool COUNTED>
__global__ __launch_bounds__(SORT_BLOCK, (sort_pass_waves<T, PERM, COUNTED>())) void sort_pass_kernel(const T* __restrict__ orig, typename SortKey<T>::U* buf_a,
                                                               typename SortKey<T>::U* buf_b, uint32_t* val_a, uint32_t* val_b,
                                                               int64_t* __restrict__ perm_out, uint32_t n, int pass, int rev, SortCtl* ctl,
                                                               uint64_t* desc, const uint32_t* __restrict__ tile_before,
                                                               const uint32_t* __restrict__ chunk_prefix, uint32_t chunk_rows,
                                                               uint32_t ntiles, long long wait_rounds, uint32_t xcd_chunk) {
    typedef typename SortKey<T>::U U;
    constexpr int TILE = SORT_BLOCK * ITEMS;
    __shared__ U lds_keys[TILE];
    __shared__ uint32_t lds_vals[PERM ? TILE : 1];
    __shared__ uint32_t cnt[SORT_NW][256];        // per wave and digit: count, then slot in the sorted tile of the wave's first key of the digit
    __shared__ uint32_t goff[256];                // global slot of the digit's first key of this tile, minus its slot in the sorted tile
    __shared__ uint32_t wsum[SORT_NW];
    __shared__ uint32_t lds_tile;

    if (ctl->skip[pass]) return;
    const bool first = (uint32_t)pass == ctl->first_pass, last = (uint32_t)pass == ctl->last_pass;
    const U umin = (U)~ctl->inv_min;
    const bool src_b = ctl->src_is_b[pass] != 0u;
    const U* in = first ? (const U*)orig : (src_b ? buf_b : buf_a);
    U* dst = src_b ? buf_a : buf_b;
    const uint32_t* vsrc = src_b ? val_b : val_a;
    uint32_t* vdst = src_b ? val_a : val_b;
    const uint32_t tag_a = ((uint32_t)(pass + 1) << 2) | 1u, tag_p = ((uint32_t)(pass + 1) << 2) | 2u;
    for (uint32_t round = 0;; ++round) {
        // everything derived from the thread's index is computed again for every tile: hoisted out of this loop it
        // would sit in some 35 registers (16 of them tid + i * 256) across the whole kernel
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        const int wave = tid / WAVE, lane = tid % WAVE;
        if (!COUNTED && tid == 0) {
            // once a look-back of this call has given up its wait the result is lost: no further tile starts
            const uint32_t failed = __hip_atomic_load(&ctl->wait_failed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t ticket = atomicAdd(&ctl->ticket[pass], 1u);
            lds_tile = failed != 0u ? ntiles : ticket;
        }
        for (int i = tid; i < SORT_NW * 256; i += SORT_BLOCK) (&cnt[0][0])[i] = 0;
        __syncthreads();
        uint32_t tile = COUNTED ? blockIdx.x + round * gridDim.x : lds_tile;
        if (COUNTED && xcd_chunk != 0u) {
            const uint32_t i = (blockIdx.x >> 3) + round * (gridDim.x >> 3);
            tile = i < xcd_chunk ? (blockIdx.x & 7u) * xcd_chunk + i : ntiles;
        }
        if (tile >= ntiles) return;
        const uint32_t e0 = tile * (uint32_t)TILE;
        const uint32_t woff = e0 + (uint32_t)wave * (WAVE * ITEMS) + lane;

        // Every tile but the last is full: its code carries no bounds checks (they cost an exec-mask save and a
        // branch per key and round).
        auto sort_tile = [&](auto full_tile) {
            constexpr bool FULL = decltype(full_tile)::value;
            // load (and map on the first pass)
            U key[ITEMS];
            uint32_t val[PERM ? ITEMS : 1];
            uint32_t rank[ITEMS];
    #pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                const uint32_t e = woff + i * WAVE;
                key[i] = (U)~(U)0;
                if (FULL || e < n) key[i] = in[e];
            }
            if constexpr (PERM) {
    #pragma unroll
                for (int i = 0; i < ITEMS; ++i) val[i] = woff + i * WAVE;              // first pass: the key's own index
                if (!first) {
    #pragma unroll
                    for (int i = 0; i < ITEMS; ++i)
                        if (FULL || woff + i * WAVE < n) val[i] = vsrc[woff + i * WAVE];
                }
            }
            if (first) {
    #pragma unroll
                for (int i = 0; i < ITEMS; ++i) key[i] = enc_bits<T>(key[i], rev, umin);    // padding keys are never counted
            }
            // rank inside the wave: lanes with the same digit find each other with 8 ballots; every lane reads the
            // wave's counter of its digit -- the rank of the group's first key -- and then the lowest lane of the group
            // adds the size of the group to it.  LDS executes the instructions of one wave in order, so the read of
            // the next round sees this add, and the 16 rounds queue up back to back; a result is used two rounds later.
            uint32_t* wcnt = cnt[wave];
            constexpr int DEPTH = 2;                       // counter reads in flight before their result is used
            uint32_t pend_before[DEPTH], pend_below[DEPTH];
    #pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                const bool valid = FULL || woff + i * WAVE < n;
                const uint32_t d = digit_of(key[i], pass);
                uint32_t same_lo, same_hi;
                match_digit_halves(d, same_lo, same_hi);
                if (!FULL) {
                    const uint64_t vm = __ballot(valid);
                    same_lo &= (uint32_t)vm;
                    same_hi &= (uint32_t)(vm >> 32);
                }
                const uint32_t below = __builtin_amdgcn_mbcnt_hi(same_hi, __builtin_amdgcn_mbcnt_lo(same_lo, 0u));
                const uint32_t before = __hip_atomic_load(&wcnt[d], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
                __builtin_amdgcn_wave_barrier();
                if (valid && below == 0u) {
                    const uint32_t total = (uint32_t)__builtin_popcount(same_lo) + (uint32_t)__builtin_popcount(same_hi);
                    __hip_atomic_fetch_add(&wcnt[d], total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
                }
                if (i >= DEPTH) rank[i - DEPTH] = pend_before[i % DEPTH] + pend_below[i % DEPTH];
                pend_before[i % DEPTH] = before;
                pend_below[i % DEPTH] = below;
                __builtin_amdgcn_sched_barrier(0);
            }
    #pragma unroll
            for (int i = ITEMS; i < ITEMS + DEPTH; ++i) rank[i - DEPTH] = pend_before[i % DEPTH] + pend_below[i % DEPTH];
            __syncthreads();
            // digit d = tid: count of the tile and of each wave
            uint32_t wave_count[SORT_NW];
            uint32_t count = 0;
    #pragma unroll
            for (int w = 0; w < SORT_NW; ++w) {
                wave_count[w] = cnt[w][tid];
                count += wave_count[w];
            }
            // publish the count, then look back over the earlier tiles for this digit
            uint64_t* my = desc + (uint64_t)tile * 256 + tid;
            uint32_t excl = 0;
            if constexpr (COUNTED) {
                excl = tile_before[(uint64_t)tile * 256 + tid] + chunk_prefix[(uint64_t)(tile / chunk_rows) * 256 + tid];
            } else if (tile == 0) {
                __hip_atomic_store(my, ((uint64_t)tag_p << 32) | count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
                __hip_atomic_store(my, ((uint64_t)tag_a << 32) | count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                // walk back over the earlier tiles, LB descriptors per round trip: sum counts until one that already
                // includes its own predecessors; a descriptor that is not written yet is polled again
                constexpr int LB = 8;
                int64_t t = (int64_t)tile - 1;
                bool done = false;
                const WaitCtl wc{&ctl->wait_failed, wait_rounds, 0, 1u};     // the control block belongs to this call alone
                long long rounds = 0;
                while (!done) {
                    uint64_t w[LB];
    #pragma unroll
                    for (int j = 0; j < LB; ++j) {
                        w[j] = ((uint64_t)tag_p << 32);                       // in front of tile 0: nothing, and final
                        if (t - j >= 0) w[j] = __hip_atomic_load(desc + (uint64_t)(t - j) * 256 + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    int j = 0;
    #pragma unroll
                    for (; j < LB; ++j) {
                        const uint32_t tg = (uint32_t)(w[j] >> 32);
                        if (tg != tag_a && tg != tag_p) break;
                        excl += (uint32_t)w[j];
                        if (tg == tag_p) { done = true; break; }
                    }
                    t -= j;
                    if (!done && j == 0) {
                        // every lane counts its own rounds (a lane per digit); one giving up makes all others follow
                        if (wait_give_up(wc, rounds)) break;
                        __builtin_amdgcn_s_sleep(2);
                    }
                }
                __hip_atomic_store(my, ((uint64_t)tag_p << 32) | (uint64_t)(excl + count), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            // first slot of every digit inside the sorted tile: exclusive scan of the counts over the 256 digits
            const uint32_t inc = wave_scan_inclusive(count, OpAdd(), 0u);
            if (lane == WAVE - 1) wsum[wave] = inc;
            __syncthreads();
            uint32_t start = inc - count;
            for (int w = 0; w < wave; ++w) start += wsum[w];
            goff[tid] = ctl->hist[pass][tid] + excl - start;
    #pragma unroll
            for (int w = 0; w < SORT_NW; ++w) {
                cnt[w][tid] = start;
                start += wave_count[w];
            }
            __syncthreads();
            // reorder the tile in LDS.  Reads first, writes after, so that the 16 table reads are in flight together.
    #pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                uint32_t d = digit_of(key[i], pass);
                asm volatile("" : "+v"(d));            // computed again here: 16 LDS addresses kept from the ranking cost a wave of occupancy
                rank[i] += wcnt[d];
            }
    #pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                if (FULL || woff + i * WAVE < n) {
                    lds_keys[rank[i]] = key[i];
                    if constexpr (PERM) lds_vals[rank[i]] = val[i];
                }
            }
            __syncthreads();
            // write runs of equal digits: thread q takes the q-th key of the sorted tile.  Again all reads of a kind
            // together; `last` is decided once, not per key.
            const uint32_t valid_n = n - e0 < (uint32_t)TILE ? n - e0 : (uint32_t)TILE;
            U out_key[ITEMS];
            uint32_t slot[ITEMS];
    #pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                const uint32_t q = (uint32_t)tid + i * SORT_BLOCK;
                out_key[i] = (U)0;
                if (FULL || q < valid_n) out_key[i] = lds_keys[q];
            }
    #pragma unroll
            for (int i = 0; i < ITEMS; ++i) slot[i] = goff[digit_of(out_key[i], pass)] + (uint32_t)tid + i * SORT_BLOCK;
            // slot < n always holds in a sound sort.  After a look-back has given up its wait (WaitCtl) the offsets are
            // too small and this pass leaves holes; the next pass then reads keys the histograms never counted, and
            // its slots can lie anywhere: keep every store inside the arrays.  (The large sorts count every tile of
            // every pass themselves and wait for nobody.)
            auto writable = [&](int i) { return (FULL || (uint32_t)tid + i * SORT_BLOCK < valid_n) && (COUNTED || slot[i] < n); };
            if constexpr (PERM) {
                uint32_t out_val[ITEMS];
    #pragma unroll
                for (int i = 0; i < ITEMS; ++i) {
                    out_val[i] = 0;
                    if (FULL || (uint32_t)tid + i * SORT_BLOCK < valid_n) out_val[i] = lds_vals[(uint32_t)tid + i * SORT_BLOCK];
                }
                if (last) {
    #pragma unroll
                    for (int i = 0; i < ITEMS; ++i) if (writable(i)) perm_out[slot[i]] = (int64_t)out_val[i] + 1;
                } else {
    #pragma unroll
                    for (int i = 0; i < ITEMS; ++i) if (writable(i)) { dst[slot[i]] = out_key[i]; vdst[slot[i]] = out_val[i]; }
                }
            } else if (last) {
    #pragma unroll
                for (int i = 0; i < ITEMS; ++i) if (writable(i)) ((T*)dst)[slot[i]] = dec_bits<T>(out_key[i], rev, umin);
            } else {
    #pragma unroll
                for (int i = 0; i < ITEMS; ++i) if (writable(i)) dst[slot[i]] = out_key[i];
            }
        };
        if (e0 + (uint32_t)TILE <= n) sort_tile(std::true_type{}); else sort_tile(std::false_type{});
        __syncthreads();      // LDS is reused by the next tile
    }
}

// ---- finish ------------------------------------------------------------------------------------------------------
// sort: after an odd number of passes the result sits in buffer B.  sortperm: no pass ran = identity permutation.
template <typename W>
__global__ __launch_bounds__(256) void sort_finish_kernel(const SortCtl* ctl, W* a, const W* b, int64_t nwords, int64_t* perm_out, int64_t n) {
    const uint32_t nexec = ctl->nexec;
    if (perm_out != nullptr) {
        if (nexec != 0u) return;
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) perm_out[i] = i + 1;
        return;
    }
    if ((nexec & 1u) == 0u) return;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nwords; i += (int64_t)gridDim.x * 256) a[i] = b[i];
}

// ---- host --------------------------------------------------------------------------------------------------------
struct SortLayout {
    size_t desc_off, clear_end, chunk_total_off, chunk_prefix_off, keys_b_off, keys_a_off, val_a_off, val_b_off, total;
    uint32_t ntiles, chunk_rows, nchunks;
    bool counted;          // large sort: desc_off holds the per-tile digit counts (uint32) instead of descriptors
};

// keys per lane and tile: 16 for every key size (8 was tried for 8-byte keys: 5.2 instead of 4.4 ms for 2^26 Float64)
constexpr int sort_items_for(size_t) { return 16; }
template <typename T> constexpr int sort_items() { return sort_items_for(sizeof(T)); }

// More tiles than this: count first, no look-back (RK_SORT_LOOKBACK_TILES).
static uint32_t sort_lookback_tiles() {
    static const uint32_t v = [] { const char* e = std::getenv("RK_SORT_LOOKBACK_TILES"); const long x = e ? std::atol(e) : 0; return x > 0 ? (uint32_t)x : 256u; }();
    return v;
}

static SortLayout sort_layout(size_t key_size, int items, int64_t n, bool perm) {
    SortLayout l{};
    const int64_t tile = (int64_t)SORT_BLOCK * items;
    l.ntiles = (uint32_t)((n + tile - 1) / tile);
    size_t off = (sizeof(SortCtl) + 255) & ~(size_t)255;
    l.counted = l.ntiles > sort_lookback_tiles();
    l.desc_off = off;
    if (l.counted) {
        l.clear_end = off;                                   // only the control block needs clearing
        off += (size_t)l.ntiles * 256 * sizeof(uint32_t);
        l.chunk_rows = (l.ntiles + TS_MAX_CHUNKS - 1) / TS_MAX_CHUNKS;
        l.nchunks = (l.ntiles + l.chunk_rows - 1) / l.chunk_rows;
        l.chunk_total_off = off;  off += (size_t)TS_MAX_CHUNKS * 256 * sizeof(uint32_t);
        l.chunk_prefix_off = off; off += (size_t)TS_MAX_CHUNKS * 256 * sizeof(uint32_t);
    } else {
        off += (size_t)l.ntiles * 256 * sizeof(uint64_t);
        l.clear_end = off;
    }
    const size_t kbytes = ((size_t)n * key_size + 255) & ~(size_t)255, vbytes = ((size_t)n * 4 + 255) & ~(size_t)255;
    l.keys_b_off = off; off += kbytes;
    if (perm) {
        l.keys_a_off = off; off += kbytes;
        l.val_a_off = off; off += vbytes;
        l.val_b_off = off; off += vbytes;
    }
    l.total = off;
    return l;
}

template <typename T>
static int32_t sort_typed(void* keys, int64_t* perm_out, int64_t n, int rev, void* tmp, size_t tmp_bytes, hipStream_t stream) {
    typedef typename SortKey<T>::U U;
    constexpr int ITEMS = sort_items<T>();
    constexpr int PASSES = (int)sizeof(T);
    const bool perm = perm_out != nullptr;
    const SortLayout l = sort_layout(sizeof(T), ITEMS, n, perm);
    if (tmp == nullptr || !is_aligned(tmp, 256) || tmp_bytes < l.total) return RK_ERR_WORKSPACE;
    char* base = (char*)tmp;
    SortCtl* ctl = (SortCtl*)base;
    uint64_t* desc = (uint64_t*)(base + l.desc_off);
    U* buf_b = (U*)(base + l.keys_b_off);
    U* buf_a = perm ? (U*)(base + l.keys_a_off) : (U*)keys;
    uint32_t* val_a = perm ? (uint32_t*)(base + l.val_a_off) : nullptr;
    uint32_t* val_b = perm ? (uint32_t*)(base + l.val_b_off) : nullptr;
    const int cus = device_info().cus;

    const int64_t init_words = (int64_t)(l.clear_end / sizeof(uint64_t));
    int64_t g = (init_words + 255) / 256;
    if (g > cus * 16) g = cus * 16;
    // floats: no read for the smallest key.  Relative keys let small-range integers skip passes (1000 .. 1255: one pass
    // instead of two); the exponent bytes of floats are constant or not whatever is subtracted, and the histograms of the
    // small sorts find constant digits by themselves.
    constexpr bool FLOAT_KEYS = !std::is_integral<T>::value;
    sort_init_kernel<<<(unsigned)g, 256, 0, stream>>>((uint64_t*)base, init_words, FLOAT_KEYS ? 1 : 0);
    RK_LAUNCH_CHECK();
    g = (n + 256 * 16 - 1) / (256 * 16);
    if (g > cus * 8) g = cus * 8;
    constexpr int KVEC = 16 / (int)sizeof(T);
    int64_t head = (int64_t)(((16 - ((uintptr_t)keys & 15)) & 15) / sizeof(T));
    if (head > n) head = n;
    const int64_t nvec = (n - head) / KVEC;
    // few workgroups: each ends with device-wide atomics on shared words (1 for the minimum, 256 per digit position)
    const unsigned gmin = (unsigned)(g < cus * 2 ? g : cus * 2), ghist = (unsigned)(g < cus * 4 ? g : cus * 4);
    // sortperm: the first pass reads the caller's keys and should write buffer A, i.e. "reads B"
    if (!l.counted) {
        if (!FLOAT_KEYS) {
            sort_min_kernel<T><<<gmin, 256, 0, stream>>>((const T*)keys, n, head, nvec, rev, ctl);
            RK_LAUNCH_CHECK();
        }
        sort_hist_kernel<T, PASSES><<<ghist, 256, 0, stream>>>((const T*)keys, n, head, nvec, rev, ctl);
        RK_LAUNCH_CHECK();
        sort_plan_kernel<<<1, 256, 0, stream>>>(ctl, PASSES, (uint32_t)n, perm ? 1 : 0, 0);
    } else if (std::is_integral<T>::value) {
        sort_minmax_kernel<T><<<gmin, MINMAX_BLOCK, 0, stream>>>((const T*)keys, n, head, nvec, rev, ctl);
        RK_LAUNCH_CHECK();
        sort_plan_kernel<<<1, 256, 0, stream>>>(ctl, PASSES, (uint32_t)n, perm ? 1 : 0, 1);
    } else {
        // floats: the digits of a large array are hardly ever constant, so no read is spent on finding out
        sort_plan_kernel<<<1, 256, 0, stream>>>(ctl, PASSES, (uint32_t)n, perm ? 1 : 0, 2);
    }
    RK_LAUNCH_CHECK();
    // tunables, read once: workgroups of the pass kernel per CU (RK_SORT_WGS_PER_CU), XCD-contiguous tiles (RK_SORT_XCD=0: off).
    // Large sorts launch one workgroup per tile unless told otherwise: the hardware's dispatcher balances the load
    // better than a fixed share of tiles per resident workgroup (2^26 Float32: 866 against 986 us with 4 a CU).
    static const int wgs_per_cu = [] { const char* e = std::getenv("RK_SORT_WGS_PER_CU"); const int x = e ? std::atoi(e) : 0; return x > 0 ? x : 0; }();
    static const int xcd_map = [] { const char* e = std::getenv("RK_SORT_XCD"); return e ? std::atoi(e) : 1; }();
    unsigned pgrid;
    if (l.counted && wgs_per_cu == 0) pgrid = (l.ntiles + 7u) & ~7u;
    else { const unsigned cap = (unsigned)(cus * (wgs_per_cu > 0 ? wgs_per_cu : 6)); pgrid = l.ntiles < cap ? l.ntiles : cap; }
    // large sorts: each XCD takes a contiguous eighth of the tiles, so the runs that neighbouring tiles write next to
    // each other meet in one L2 (workgroups go to the XCDs round-robin by their index)
    const uint32_t xcd_chunk = (xcd_map != 0 && l.counted && pgrid % 8u == 0u) ? (l.ntiles + 7u) / 8u : 0u;
    uint32_t* tile_count = (uint32_t*)desc;
    uint32_t* chunk_total = l.counted ? (uint32_t*)(base + l.chunk_total_off) : nullptr;
    uint32_t* chunk_prefix = l.counted ? (uint32_t*)(base + l.chunk_prefix_off) : nullptr;
    const long long wb = wait_budget();
    for (int p = 0; p < PASSES; ++p) {
        if (l.counted) {
            sort_upsweep_kernel<T, ITEMS><<<l.ntiles, SORT_BLOCK, 0, stream>>>((const T*)keys, buf_a, buf_b, (uint32_t)n, p, rev, ctl, tile_count);
            RK_LAUNCH_CHECK();
            sort_tilescan_kernel<<<l.nchunks, TS_BLOCK, 0, stream>>>(ctl, p, tile_count, l.ntiles, l.chunk_rows, chunk_total, chunk_prefix);
            RK_LAUNCH_CHECK();
            if (perm) sort_pass_kernel<T, ITEMS, true, true><<<pgrid, SORT_BLOCK, 0, stream>>>((const T*)keys, buf_a, buf_b, val_a, val_b, perm_out, (uint32_t)n, p, rev, ctl, desc, tile_count, chunk_prefix, l.chunk_rows, l.ntiles, wb, xcd_chunk);
            else sort_pass_kernel<T, ITEMS, false, true><<<pgrid, SORT_BLOCK, 0, stream>>>((const T*)keys, buf_a, buf_b, nullptr, nullptr, nullptr, (uint32_t)n, p, rev, ctl, desc, tile_count, chunk_prefix, l.chunk_rows, l.ntiles, wb, xcd_chunk);
        } else {
            if (perm) sort_pass_kernel<T, ITEMS, true, false><<<pgrid, SORT_BLOCK, 0, stream>>>((const T*)keys, buf_a, buf_b, val_a, val_b, perm_out, (uint32_t)n, p, rev, ctl, desc, nullptr, nullptr, 1u, l.ntiles, wb, 0u);
            else sort_pass_kernel<T, ITEMS, false, false><<<pgrid, SORT_BLOCK, 0, stream>>>((const T*)keys, buf_a, buf_b, nullptr, nullptr, nullptr, (uint32_t)n, p, rev, ctl, desc, nullptr, nullptr, 1u, l.ntiles, wb, 0u);
        }
        RK_LAUNCH_CHECK();
    }
    const int64_t nwords = ((int64_t)n * (int64_t)sizeof(T) + 3) / 4;
    g = ((perm ? n : nwords) + 255) / 256;
    if (g > cus * 16) g = cus * 16;
    // whole 32-bit words: buffers are 256-byte padded, the caller's array is at least element-aligned; 16-bit keys
    // with an odd count copy one element more than n only inside buffer padding on the source side -- so copy by element there
    if (sizeof(T) == 2) sort_finish_kernel<uint16_t><<<(unsigned)g, 256, 0, stream>>>(ctl, (uint16_t*)keys, (const uint16_t*)buf_b, perm ? 0 : n, perm_out, n);
    else sort_finish_kernel<uint32_t><<<(unsigned)g, 256, 0, stream>>>(ctl, (uint32_t*)keys, (const uint32_t*)buf_b, perm ? 0 : nwords, perm_out, n);
    RK_LAUNCH_CHECK();
    return RK_SUCCESS;
}

static bool sort_dtype_size(int dt, size_t* size) {
    switch (dt) {
        case RK_F32: case RK_I32: *size = 4; return true;
        case RK_F64: case RK_I64: *size = 8; return true;
        case RK_F16: case RK_I16: *size = 2; return true;
        default: return false;
    }
}

}  // namespace rk

using namespace rk;

extern "C" size_t rk_sort_tmp_bytes(rk_dtype dt, int64_t n, int32_t with_perm) {
    size_t ks = 0;
    if (!sort_dtype_size((int)dt, &ks) || n <= 0) return 256;
    return sort_layout(ks, sort_items_for(ks), n, with_perm != 0).total;
}

static int32_t sort_dispatch(rk_dtype dt, void* keys, int64_t* perm_out, int64_t n, int32_t rev, void* tmp, size_t tmp_bytes, void* stream) {
    size_t ks = 0;
    if (!sort_dtype_size((int)dt, &ks)) return ((int)dt >= RK_F32 && (int)dt <= RK_I16) ? RK_ERR_UNSUPPORTED : RK_ERR_INVALID_ARGUMENT;
    if (n < 0) return RK_ERR_INVALID_ARGUMENT;
    if (n == 0) return RK_SUCCESS;
    if (keys == nullptr || !is_aligned(keys, ks)) return RK_ERR_INVALID_ARGUMENT;
    if (n >= ((int64_t)1 << 31)) return RK_ERR_TOO_LARGE;
    hipStream_t st = (hipStream_t)stream;
    const int r = (rev ? SORT_REV : 0) | (perm_out == nullptr ? SORT_KEEP_NAN : 0);
    switch ((int)dt) {
        case RK_F32: return sort_typed<float>(keys, perm_out, n, r, tmp, tmp_bytes, st);
        case RK_F64: return sort_typed<double>(keys, perm_out, n, r, tmp, tmp_bytes, st);
        case RK_I32: return sort_typed<int32_t>(keys, perm_out, n, r, tmp, tmp_bytes, st);
        case RK_I64: return sort_typed<int64_t>(keys, perm_out, n, r, tmp, tmp_bytes, st);
        case RK_F16: return sort_typed<half_bits>(keys, perm_out, n, r, tmp, tmp_bytes, st);
        default:     return sort_typed<int16_t>(keys, perm_out, n, r, tmp, tmp_bytes, st);
    }
}

extern "C" int32_t rk_sort_status(const void* tmp, size_t tmp_bytes, void* stream) {
    if (tmp == nullptr) return RK_ERR_INVALID_ARGUMENT;
    if (!is_aligned(tmp, 256) || tmp_bytes < sizeof(SortCtl)) return RK_ERR_WORKSPACE;
    uint32_t failed = 0;
    RK_HIP(hipMemcpyAsync(&failed, (const char*)tmp + offsetof(SortCtl, wait_failed), sizeof(failed), hipMemcpyDeviceToHost, (hipStream_t)stream));
    RK_HIP(hipStreamSynchronize((hipStream_t)stream));
    return failed != 0u ? RK_ERR_WAIT : RK_SUCCESS;
}

extern "C" int32_t rk_sort(rk_dtype dt, void* keys, int64_t n, int32_t rev, void* tmp, size_t tmp_bytes, void* stream) {
    return sort_dispatch(dt, keys, nullptr, n, rev, tmp, tmp_bytes, stream);
}

extern "C" int32_t rk_sortperm(rk_dtype dt, const void* keys, int64_t* perm_out, int64_t n, int32_t rev, void* tmp, size_t tmp_bytes,
                               void* stream) {
    if (n > 0 && perm_out == nullptr) return RK_ERR_INVALID_ARGUMENT;
    return sort_dispatch(dt, (void*)keys, perm_out, n, rev, tmp, tmp_bytes, stream);
}
