// findall(::ROCArray{Bool}) in one pass over the mask: stream compaction with the chained look-back of the
// scan.  Replaces the cumsum + `_ker!` pair of src/kernels/indexing.jl:8-36 (9 bytes per element for the Int64
// cumsum, 9 more for the scatter) by 1 byte per element read plus the indices written.
#include <cstdlib>

#include "rk_common.hpp"
#include "rk_scan_impl.hpp"

namespace rk {

constexpr int SEL_CHUNK = WAVE * 16;                         // Bools one wave covers with one 16-byte load per lane

struct SelShape {
    int64_t s[RK_MAX_DIMS];
    int ndim;
};

// Writes the 1-based index of element `i` (0-based, column-major) as entry `pos` of ys.
template <bool LINEAR, bool SMALL>
__device__ __forceinline__ void emit_index(int64_t* __restrict__ ys, int64_t pos, int64_t i, const SelShape& shp) {
    if constexpr (LINEAR) {
        ys[pos] = i + 1;
    } else if constexpr (SMALL) {                            // every extent and the length fit 32 bits
        uint32_t rem = (uint32_t)i;
        for (int d = 0; d < shp.ndim; ++d) {
            const uint32_t e = (uint32_t)shp.s[d], q = rem / e;
            ys[pos * shp.ndim + d] = (int64_t)(rem - q * e) + 1;
            rem = q;
        }
    } else {
        int64_t rem = i;
        for (int d = 0; d < shp.ndim; ++d) {
            const int64_t q = rem / shp.s[d];
            ys[pos * shp.ndim + d] = rem - q * shp.s[d] + 1;
            rem = q;
        }
    }
}

// Persistent workgroups take tiles of SEL_NW * SEL_K * 1024 Bools in acquisition order (see scan_chain_kernel).
// A lane counts the set bytes of its SEL_K 16-byte loads, the counts are scanned across the wave (DPP) and the
// workgroup (LDS), the tile total is published and the tile's offset resolved by the two-level look-back.
// Output: per load, the lanes drop the in-chunk offsets of their set bytes into the wave's LDS strip at their
// scanned positions; the wave then reads the strip back in order and writes indices with coalesced stores (a
// lane writing its own run directly makes every store instruction touch 64 different lines: 4x slower at high
// density).  Only bit 0 of a byte is looked at (Julia's Bool).
// ORDERED: one workgroup per tile (its number from the launch order or, for grids beyond what is resident at once, from the
// counter: ordered_tile_id), the look-back and the end of the call as in scan_ordered_kernel
// (no tile counter, only the first tile of a group of 64 reads group descriptors, each on a line of its own).
// Set bytes of another tile, counted by the calling wave (the look-back's way out when that tile's workgroup is not
// there to publish its count: desc_lookback_alone).  Every tile in front of another is full.
template <int SEL_TILE> struct SelectTileCount {
    const uint8_t* bools;
    int aligned;
    __device__ __forceinline__ int64_t operator()(int64_t p) const {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const uint8_t* q = bools + p * (int64_t)SEL_TILE;
        int32_t c = 0;
        for (int i = lane_id() * 16; i < SEL_TILE; i += WAVE * 16) {
            if (aligned) {
                const u32x4 x = *(const u32x4*)(q + i) & 0x01010101u;
                c += __popc(x[0]) + __popc(x[1]) + __popc(x[2]) + __popc(x[3]);
            } else {
                for (int b = 0; b < 16; ++b) c += q[i + b] & 1;
            }
        }
        return (int64_t)wave_reduce(c, OpAdd());
    }
};

template <bool LINEAR, bool SMALL, int SEL_NW, int SEL_K, bool ORDERED>
__global__ __launch_bounds__(SEL_NW * WAVE) void findall_select_kernel(const uint8_t* __restrict__ bools, int64_t n, int64_t* __restrict__ ys,
                                                                       int64_t* __restrict__ count_out, SelShape shp, int aligned,
                                                                       unsigned long long* counter, uint32_t* tickets, int ticket_group,
                                                                       uint64_t* desc, int64_t ntiles, int64_t ngroups, int64_t desc_capacity,
                                                                       WaitCtl wc, WaitAlone wa, int dynamic_ids) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    constexpr int SEL_TILE = SEL_NW * SEL_CHUNK * SEL_K;
    __shared__ uint16_t lds_strip[SEL_NW][SEL_CHUNK];
    __shared__ int32_t lds_wave[SEL_NW];
    __shared__ int64_t lds_prefix;
    __shared__ unsigned long long lds_id;
    const int tid = threadIdx.x, wave = tid / WAVE, lane = lane_id();
    uint64_t* tile_desc = desc;                                          // [2 words][ntiles]
    uint64_t* group_desc = desc + (int64_t)Words<int64_t>::N * ntiles;   // [2 words][ngroups]; ORDERED: a line per group
    const OpAdd op;

    unsigned long long cur;
    if constexpr (ORDERED) {
        const OrderedId id = ordered_tile_id(counter, dynamic_ids, true);
        cur = ((unsigned long long)id.epoch << 32) | (unsigned long long)id.tile;
    } else {
        if (tid == 0) lds_id = __hip_atomic_fetch_add(counter, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        cur = lds_id;
    }
    while ((int64_t)(cur & 0xffffffffull) < ntiles) {
        const int64_t tile = (int64_t)(cur & 0xffffffffull);
        const uint32_t epoch = (uint32_t)(cur >> 32);
        wc.stamp = epoch;
        const int64_t e0 = tile * SEL_TILE;
        const int64_t left = n - e0;
        const int valid = left < SEL_TILE ? (int)left : SEL_TILE;
        const int woff = wave * (SEL_CHUNK * SEL_K) + lane * 16;
        // per 16-byte load: bit b of `hits` = byte b of the lane's 16 is set; `pk` packs the lane's first output
        // position inside the chunk (high half) with the hits (low half), so a tile costs one register per load
        uint32_t pk[SEL_K];
        int32_t ktot[SEL_K];                     // hits of the whole chunk (wave-uniform)
        int32_t carry = 0;
#pragma unroll
        for (int k0 = 0; k0 < SEL_K; k0 += 4) {
            u32x4 x[4];
            if (aligned && valid == SEL_TILE) {
#pragma unroll
                for (int k = 0; k < 4; ++k) x[k] = load_nt((const u32x4*)(bools + e0 + woff + (k0 + k) * SEL_CHUNK));
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        uint32_t word = 0;
#pragma unroll
                        for (int b = 0; b < 4; ++b) {
                            const int idx = woff + (k0 + k) * SEL_CHUNK + q * 4 + b;
                            if (idx < valid) word |= (uint32_t)bools[e0 + idx] << (8 * b);
                        }
                        x[k][q] = word;
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < 4; k += 2) {
                // bit 0 of the 16 bytes -> a 16-bit mask in memory order: a dot product of the four bytes of a word with
                // (1, 2, 4, 8) or (16, 32, 64, 128) gathers four of them (a 32-bit multiply does too, at a quarter of
                // the rate).  The counts of two loads share one scan across the wave (a chunk holds at most 1024 hits).
                uint32_t hits[2];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const u32x4 b = x[k + h] & 0x01010101u;
                    const uint32_t lo = __builtin_amdgcn_udot4(b[1], 0x80402010u, __builtin_amdgcn_udot4(b[0], 0x08040201u, 0u, false), false);
                    const uint32_t hi = __builtin_amdgcn_udot4(b[3], 0x80402010u, __builtin_amdgcn_udot4(b[2], 0x08040201u, 0u, false), false);
                    hits[h] = lo | (hi << 8);
                }
                const int32_t c = (int32_t)(__popc(hits[0]) | ((uint32_t)__popc(hits[1]) << 16));
                const int32_t inc = wave_scan_inclusive(c, op, 0);
                const uint32_t exc = (uint32_t)(inc - c);
                pk[k0 + k] = (exc << 16) | hits[0];
                pk[k0 + k + 1] = (exc & 0xffff0000u) | hits[1];
                const uint32_t tot = (uint32_t)read_lane(inc, WAVE - 1);
                ktot[k0 + k] = (int32_t)(tot & 0xffffu);
                ktot[k0 + k + 1] = (int32_t)(tot >> 16);
                carry += ktot[k0 + k] + ktot[k0 + k + 1];
            }
        }
        if (lane == 0) lds_wave[wave] = carry;
        __syncthreads();
        int32_t wave_prefix = 0, tile_count = 0;
#pragma unroll
        for (int w = 0; w < SEL_NW; ++w) {
            const int32_t c = lds_wave[w];
            if (w < wave) wave_prefix += c;
            tile_count += c;
        }
        if (wave == 0) {
            int64_t tile_prefix = 0;
            if (lane == 0) desc_publish(tile_desc, ntiles, tile, (int64_t)tile_count, (epoch << 2) | DESC_A);
            if (tile > 0) {
                if constexpr (ORDERED) {
                    bool expired = false;
                    tile_prefix = desc_lookback_leader(tile_desc, ntiles, group_desc, tile, tile, tile >> 6, epoch, (int64_t)tile_count,
                                                       (int64_t)0, op, (int64_t)0, wc, wa, expired);
                    if (expired)
                        tile_prefix = desc_lookback_alone(tile_desc, ntiles, group_desc, tile, tile, tile >> 6, epoch, (int64_t)tile_count,
                                                          (int64_t)0, op, (int64_t)0, SelectTileCount<SEL_TILE>{bools, aligned}, wa.counter);
                } else
                    tile_prefix = desc_lookback2(tile_desc, ntiles, group_desc, ngroups, tile, tile, tile >> 6, epoch, (int64_t)tile_count,
                                                 (int64_t)0, op, (int64_t)0, wc);
            }
            if (lane == 0) {
                lds_prefix = tile_prefix;
                if (tile == ntiles - 1 && count_out != nullptr) *count_out = tile_prefix + tile_count;
            }
        }
        __syncthreads();
        int64_t base = lds_prefix + wave_prefix;
        // The hits of consecutive chunks share the strip while they fit (SEL_CHUNK entries; an entry is an offset from
        // the first chunk of the batch, < 16 * 1024): a sparse mask leaves in one round per wave instead of one per
        // chunk, each of which costs two LDS round trips.  fill, kbase: wave-uniform.
        uint16_t* strip = lds_strip[wave];
        int32_t fill = 0, kbase = 0;
        auto flush = [&]() {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            const int64_t i0 = e0 + wave * (SEL_CHUNK * SEL_K) + kbase * SEL_CHUNK;
            for (int i = lane; i < fill; i += WAVE) emit_index<LINEAR, SMALL>(ys, base + i, i0 + strip[i], shp);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();                              // the strip is reused by the next batch
            base += fill;
            fill = 0;
        };
#pragma unroll
        for (int k = 0; k < SEL_K; ++k) {
            if (ktot[k] == 0) continue;                                   // wave-uniform
            if (fill + ktot[k] > SEL_CHUNK) flush();
            if (fill == 0) kbase = k;
            int32_t p = fill + (int32_t)(pk[k] >> 16);
            const uint32_t rel = (uint32_t)((k - kbase) * SEL_CHUNK + lane * 16 - 1);
            for (uint32_t m = pk[k] & 0xffffu; m != 0u; m &= m - 1u) strip[p++] = (uint16_t)(rel + __ffs(m));
            fill += ktot[k];
        }
        if (fill > 0) flush();
        if constexpr (ORDERED) break;
        if (tid == 0) lds_id = __hip_atomic_fetch_add(counter, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        cur = lds_id;
    }
    if constexpr (ORDERED)
        ordered_finish((uint32_t)(cur >> 32), (int64_t)Words<int64_t>::N * ntiles + ngroups * GROUP_DESC_STRIDE, counter, tickets, ticket_group,
                       desc, desc_capacity);
    else
        chain_finish(cur, ntiles, (int64_t)Words<int64_t>::N * (ntiles + ngroups), counter, desc, desc_capacity);
}

__global__ void store_count_kernel(int64_t* p, int64_t v) { *p = v; }

// 16-byte loads per lane and tile (RK_SELECT_LOADS: 4, 8 or 16).  Measured on MI355X, 2^28 Bools, 1 % / 25 % / 100 %
// set, 8 waves in launch order: 4 loads 112 / 188 / 425 us, 8 loads 78 / 167 / 462 us, 16 loads 63 / 159 / 473 us: every
// tile costs about 10 ns whatever feeds it, so larger tiles win until the output dominates.
int tune_select_loads() {
    static const int v = [] { const char* s = std::getenv("RK_SELECT_LOADS"); const int x = s ? std::atoi(s) : 0; return (x == 4 || x == 8 || x == 16) ? x : 16; }();
    return v;
}
int tune_select_tile_ki() {
    static const int v = [] { const char* s = std::getenv("RK_SELECT_TILE_KI"); const int x = s ? std::atoi(s) : 0; return (x == 32 || x == 64 || x == 128) ? x : 0; }();
    return v;
}
int tune_select_blocks_per_cu() {
    static const int v = [] { const char* s = std::getenv("RK_SELECT_BLOCKS_PER_CU"); const int x = s ? std::atoi(s) : 0; return (x >= 1 && x <= 2) ? x : 2; }();
    return v;
}

// One workgroup of 8 waves per tile in launch order (1), or persistent workgroups of 16 waves fed by a tile counter (0).
// 2^26 / 2^28 Bools, 1 % / 25 % / 100 % set, 16 loads: ordered 22.7 / 39.4 / 122 us and 63 / 159 / 473 us, counter-fed
// 24.1 / 40.8 / 118 and 69 / 168 / 460 us (four workgroups a compute unit overlap their phases better than two; the
// look-back itself was not the limit: 16 waves in launch order measured 25 / 42 / 123 us).
int tune_select_ordered() {
    static const int v = [] { const char* s = std::getenv("RK_SELECT_ORDERED"); return s ? std::atoi(s) : 1; }();
    return v;
}

size_t findall_workspace_need(int64_t n) {
    const int64_t SEL_TILE = 8 * SEL_CHUNK * 4;                            // the smallest tile any configuration uses
    const int64_t ntiles = (n + SEL_TILE - 1) / SEL_TILE, ngroups = (ntiles + WAVE - 1) / WAVE;
    return ((size_t)ntiles * Words<int64_t>::N + (size_t)ngroups * GROUP_DESC_STRIDE) * sizeof(uint64_t);   // the ordered layout, the larger
}

}  // namespace rk

using namespace rk;

extern "C" int32_t rk_findall(const uint8_t* bools, int ndim, const int64_t* shape, int64_t* ys, int64_t* count_out, void* ws,
                              size_t ws_bytes, void* stream) {
    if (ndim < 0 || ndim > RK_MAX_DIMS || (ndim > 0 && shape == nullptr)) return RK_ERR_INVALID_ARGUMENT;
    SelShape shp{};
    shp.ndim = ndim;
    int64_t n = 1;
    bool small = true;
    for (int d = 0; d < RK_MAX_DIMS; ++d) {
        shp.s[d] = d < ndim ? shape[d] : 1;
        if (shp.s[d] < 0) return RK_ERR_INVALID_ARGUMENT;
        if (shp.s[d] != 0 && n > INT64_MAX / shp.s[d]) return RK_ERR_INVALID_ARGUMENT;
        n *= shp.s[d];
    }
    if (n == 0) {
        if (count_out != nullptr) {
            store_count_kernel<<<1, 1, 0, (hipStream_t)stream>>>(count_out, 0);
            RK_LAUNCH_CHECK();
        }
        return RK_SUCCESS;
    }
    if (bools == nullptr || ys == nullptr) return RK_ERR_INVALID_ARGUMENT;
    if (n > 0xffffffffll) small = false;
    const bool ordered = tune_select_ordered() != 0;
    int nw = 16, kl = tune_select_loads();
    if (ordered) {
        // Tiles of 32, 64 or 128 Ki Bools (RK_SELECT_TILE_KI forces one): a small mask in large tiles leaves most compute
        // units idle behind a chain of a few tiles.  25 % set, back to back: 2^21 Bools 9.6 / 12.1 / 16.5 us, 2^24
        // 17.0 / 17.7 / 22.7, 2^25 24.2 / 24.0 / 24.7, 2^26 43.7 / 44.1 / 39.2, 2^27 89.9 / 87.6 / 82.8 (16 Ki: no better)
        int ki = tune_select_tile_ki();
        if (ki == 0) ki = n <= ((int64_t)1 << 24) ? 32 : n <= ((int64_t)1 << 25) ? 64 : 128;
        nw = 8;
        kl = ki == 128 ? 16 : ki == 64 ? 8 : 4;
    }
    const int64_t SEL_TILE = (int64_t)nw * SEL_CHUNK * kl;
    const int64_t ntiles = (n + SEL_TILE - 1) / SEL_TILE, ngroups = (ntiles + WAVE - 1) / WAVE;
    if (ntiles > 0x3fffffff) return RK_ERR_TOO_LARGE;
    Workspace w{};
    if (!carve_workspace(ws, ws_bytes, findall_workspace_need(n), &w)) return RK_ERR_WORKSPACE;
    const int64_t cap = (int64_t)(w.desc_bytes / sizeof(uint64_t));
    int64_t grid = (int64_t)device_info().cus * tune_select_blocks_per_cu();
    if (grid > ntiles || ordered) grid = ntiles;
    const int tg = ordered_ticket_group(ntiles);
    unsigned long long* counter = (unsigned long long*)&w.hdr->scan_counter;
    const int aligned = is_aligned(bools, 16) ? 1 : 0;
    const WaitCtl wc = wait_ctl(w.hdr);
    const int dyn = ordered ? ordered_dynamic_ids(ntiles, nw * WAVE, true) : 0;
    hipStream_t st = (hipStream_t)stream;
#define RK_SELECT3(LIN, SM, NWW, KK, ORD)                                                                                        \
    findall_select_kernel<LIN, SM, NWW, KK, ORD><<<(unsigned)grid, NWW * WAVE, 0, st>>>(bools, n, ys, count_out, shp, aligned,      \
                                                                                        counter, w.tickets, tg, w.desc, ntiles,    \
                                                                                        ngroups, cap, wc, wait_alone(w.hdr), dyn)
#define RK_SELECT2(LIN, SM, KK)                                                                                                  \
    do {                                                                                                                         \
        if (!ordered) RK_SELECT3(LIN, SM, 16, KK, false);                                                                        \
        else RK_SELECT3(LIN, SM, 8, KK, true);                                                                                   \
    } while (0)
#define RK_SELECT(LIN, SM)                                                                                                       \
    do {                                                                                                                         \
        if (kl == 4) RK_SELECT2(LIN, SM, 4);                                                                                     \
        else if (kl == 8) RK_SELECT2(LIN, SM, 8);                                                                                \
        else RK_SELECT2(LIN, SM, 16);                                                                                            \
    } while (0)
    if (ndim <= 1) RK_SELECT(true, true);
    else if (small) RK_SELECT(false, true);
    else RK_SELECT(false, false);
#undef RK_SELECT
#undef RK_SELECT2
#undef RK_SELECT3
    RK_LAUNCH_CHECK();
    return RK_SUCCESS;
}

// ---- x[.., indices]: the gather behind logical indexing ------------------------------------------------------------
// y[i, j] = x[i, idx[j] - 1] for i < inner: `x[mask]`, `x[:, mask]`, `x[:, :, mask]` (test/hip_rocarray/indexing.jl:5-18)
// after Base.to_index has turned the mask into findall(mask) (src/kernels/indexing.jl:1).  Elements are opaque.
namespace rk {

template <typename E> struct GatherElem { typedef E type; };
struct Bytes16 { uint64_t lo, hi; };

template <typename E>
__global__ __launch_bounds__(256) void gather_slices_kernel(const E* __restrict__ x, const int64_t* __restrict__ idx, E* __restrict__ y,
                                                            int64_t inner, int64_t total, int64_t nsrc) {
    const int64_t f = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (f >= total) return;
    int64_t i = 0, j = f;
    if (inner != 1) { j = f / inner; i = f - j * inner; }
    const int64_t s = idx[j] - 1;
    if (s < 0 || s >= nsrc) return;          // an index outside x selects nothing (the caller checks bounds)
    y[f] = x[s * inner + i];
}

}  // namespace rk

extern "C" int32_t rk_gather_slices(const void* x, const int64_t* idx, void* y, size_t elsize, int64_t inner, int64_t nidx, int64_t nsrc,
                                    void* stream) {
    if (inner < 0 || nidx < 0 || nsrc < 0) return RK_ERR_INVALID_ARGUMENT;
    if (elsize != 1 && elsize != 2 && elsize != 4 && elsize != 8 && elsize != 16) return RK_ERR_UNSUPPORTED;
    if (inner == 0 || nidx == 0) return RK_SUCCESS;
    if (x == nullptr || idx == nullptr || y == nullptr) return RK_ERR_INVALID_ARGUMENT;
    const size_t align = elsize < 16 ? elsize : 8;
    if (!is_aligned(x, align) || !is_aligned(y, align)) return RK_ERR_INVALID_ARGUMENT;
    if (nidx > INT64_MAX / inner) return RK_ERR_TOO_LARGE;
    const int64_t total = inner * nidx, blocks = (total + 255) / 256;
    if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
    hipStream_t st = (hipStream_t)stream;
#define RK_GATHER(E) rk::gather_slices_kernel<E><<<(unsigned)blocks, 256, 0, st>>>((const E*)x, idx, (E*)y, inner, total, nsrc)
    switch (elsize) {
        case 1: RK_GATHER(uint8_t); break;
        case 2: RK_GATHER(uint16_t); break;
        case 4: RK_GATHER(uint32_t); break;
        case 8: RK_GATHER(uint64_t); break;
        default: RK_GATHER(rk::Bytes16); break;
    }
#undef RK_GATHER
    RK_LAUNCH_CHECK();
    return RK_SUCCESS;
}
