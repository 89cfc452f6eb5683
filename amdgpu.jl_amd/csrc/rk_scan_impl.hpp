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
//   scan_thread_kernel         one lane per line (tiny lines / narrow inner)
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

// Exclusive prefix of `tile` inside its line; executed by one full wave, result wave-uniform.
// `tl` = number of predecessors the tile has in its line.
template <typename T, typename Op>
__device__ __forceinline__ T desc_lookback(const uint64_t* desc, int64_t stride, int64_t tile, int64_t tl, uint32_t epoch,
                                           Op op, T ident) {
    const int lane = lane_id();
    const uint32_t tagA = (epoch << 2) | DESC_A, tagP = (epoch << 2) | DESC_P;
    T prefix = ident;
    int64_t first = tile - 1;   // nearest predecessor of the current window
    int64_t remaining = tl;
    while (true) {
        const bool in_line = lane < remaining;
        const int64_t p = first - lane;
        uint32_t status;
        Words<T> val;
        int np;
        while (true) {
            if (in_line) {
                status = 0;
#pragma unroll
                for (int i = 0; i < Words<T>::N; ++i) {
                    const uint64_t d = __hip_atomic_load(&desc[i * stride + p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const uint32_t tag = (uint32_t)(d >> 32);
                    val.w[i] = (uint32_t)d;
                    const uint32_t st = tag == tagA ? DESC_A : (tag == tagP ? DESC_P : 0u);
                    status = (i == 0) ? st : (st == status ? st : 0u);
                }
            } else {            // before the start of the line: terminates the search
                status = DESC_P;
                val = to_words(ident);
            }
            const uint64_t ballotP = __ballot(status == DESC_P);
            const uint64_t ballotX = __ballot(status == 0u);
            np = ballotP ? (__ffsll((unsigned long long)ballotP) - 1) : -1;
            const uint64_t needed = np >= 0 ? ((1ull << np) - 1ull) : ~0ull;
            if ((ballotX & needed) == 0) break;
            __builtin_amdgcn_s_sleep(1);
        }
        const T x = (np < 0 || lane <= np) ? from_words<T>(val) : ident;
        prefix = op(wave_reduce(x, op), prefix);
        if (np >= 0) break;
        first -= WAVE;
        remaining -= WAVE;
    }
    return prefix;
}

struct ScanGeom {
    int64_t inner, mid, outer;
};

// ---- contiguous lines, tiles with look-back ------------------------------------------------------
template <typename In, typename T, typename Op, bool VECTOR, bool LOOKBACK, int BLOCK, int K>
__global__ __launch_bounds__(BLOCK) void scan_lookback_kernel(const In* __restrict__ in, T* __restrict__ out, int64_t line_len,
                                                              int64_t tiles_per_line, int64_t ntiles, T init, int inclusive,
                                                              Op op, WsHeader* hdr, uint64_t* desc, int64_t desc_stride,
                                                              int64_t desc_capacity) {
    constexpr int VEC = 16 / sizeof(T);
    constexpr int NW = BLOCK / WAVE;
    constexpr int WAVE_ELEMS = WAVE * VEC * K;
    constexpr int TILE = NW * WAVE_ELEMS;
    typedef typename VecOf<T, VEC>::type VT;
    typedef typename VecOf<In, VEC>::type VI;
    __shared__ T lds_wave[NW];
    __shared__ T lds_prefix;
    __shared__ uint32_t lds_tile, lds_epoch;

    const T ident = Op::template identity<T>();
    const int tid = threadIdx.x, wave = tid / WAVE, lane = lane_id();
    int64_t tile;
    uint32_t epoch = 0;
    if constexpr (LOOKBACK) {
        // tile ids in start order: every predecessor of a tile is already running or finished
        if (tid == 0) {
            lds_tile = __hip_atomic_fetch_add(&hdr->tile_counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            lds_epoch = __hip_atomic_load(&hdr->epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        tile = lds_tile;
        epoch = lds_epoch;
    } else {
        tile = blockIdx.x;
    }
    const int64_t line = tile / tiles_per_line, tl = tile - line * tiles_per_line;
    const int64_t e0 = line * line_len + tl * TILE;
    const int64_t left = line_len - tl * TILE;
    const int valid = left < TILE ? (int)left : TILE;
    const int woff = wave * WAVE_ELEMS + lane * VEC;

    T v[K][VEC];
    if (VECTOR && valid == TILE) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const VI x = load_nt((const VI*)(in + e0 + woff + k * WAVE * VEC));
            if constexpr (VEC == 1) v[k][0] = (T)x;
            else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[k][j] = (T)x[j];
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const int idx = woff + k * WAVE * VEC + j;
                v[k][j] = idx < valid ? (T)in[e0 + idx] : ident;
            }
    }

    // scan inside the thread, then across the wave, carrying the running total from load k to k+1
    T excl[K];
    T carry = ident;
#pragma unroll
    for (int k = 0; k < K; ++k) {
#pragma unroll
        for (int j = 1; j < VEC; ++j) v[k][j] = op(v[k][j - 1], v[k][j]);
        const T inc = wave_scan_inclusive(v[k][VEC - 1], op, ident);
        excl[k] = op(carry, wave_shift_right(inc, ident));
        carry = op(carry, read_lane(inc, WAVE - 1));
    }
    if (lane == 0) lds_wave[wave] = carry;
    __syncthreads();
    T wave_prefix = ident, tile_agg = ident;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        const T x = lds_wave[w];
        if (w < wave) wave_prefix = op(wave_prefix, x);
        tile_agg = op(tile_agg, x);
    }

    T tile_prefix = init;
    if constexpr (LOOKBACK) {
        if (wave == 0) {
            if (tl == 0) {
                if (lane == 0) desc_publish(desc, desc_stride, tile, op(init, tile_agg), (epoch << 2) | DESC_P);
            } else {
                if (lane == 0) desc_publish(desc, desc_stride, tile, tile_agg, (epoch << 2) | DESC_A);
                // the chain of aggregates always ends at an inclusive prefix (tile 0 of the line
                // publishes one directly), which already contains init
                tile_prefix = desc_lookback(desc, desc_stride, tile, tl, epoch, op, ident);
                if (lane == 0) desc_publish(desc, desc_stride, tile, op(tile_prefix, tile_agg), (epoch << 2) | DESC_P);
            }
            if (lane == 0) lds_prefix = tile_prefix;
        }
        __syncthreads();
        tile_prefix = lds_prefix;
    }
    const T base = op(tile_prefix, wave_prefix);

    if (VECTOR && valid == TILE) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const T off = op(base, excl[k]);
            VT o;
            if constexpr (VEC == 1) o = inclusive ? op(off, v[k][0]) : off;
            else {
                if (inclusive) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) o[j] = op(off, v[k][j]);
                } else {
                    o[0] = off;
#pragma unroll
                    for (int j = 1; j < VEC; ++j) o[j] = op(off, v[k][j - 1]);
                }
            }
            store_nt((VT*)(out + e0 + woff + k * WAVE * VEC), o);
        }
    } else {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const T off = op(base, excl[k]);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const int idx = woff + k * WAVE * VEC + j;
                if (idx < valid) out[e0 + idx] = inclusive ? op(off, v[k][j]) : (j == 0 ? off : op(off, v[k][j - 1]));
            }
        }
    }

    if constexpr (LOOKBACK) {
        // Only wave 0 touches the descriptors; once it has published, this tile is done with them.
        if (wave == 0) {
            uint32_t old = 0;
            if (lane == 0) old = __hip_atomic_fetch_add(&hdr->done_counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            old = (uint32_t)__builtin_amdgcn_readfirstlane((int)old);
            if (old == (uint32_t)ntiles - 1u) {
                // last tile of the call: leave counters clean, move to the next generation
                if (epoch >= WS_EPOCH_LAST) {
                    for (int64_t i = lane; i < desc_capacity; i += WAVE) desc[i] = 0;
                    if (lane == 0) hdr->epoch = WS_EPOCH_FIRST;
                } else if (lane == 0) hdr->epoch = epoch + 1;
                if (lane == 0) { hdr->tile_counter = 0; hdr->done_counter = 0; }
            }
        }
    }
}


// ---- contiguous lines shorter than a tile: one wave per line -------------------------------------
template <typename In, typename T, typename Op, bool VECTOR, int BLOCK>
__global__ __launch_bounds__(BLOCK) void scan_wave_lines_kernel(const In* __restrict__ in, T* __restrict__ out, int64_t line_len,
                                                                int64_t nlines, T init, int inclusive, Op op) {
    constexpr int VEC = VECTOR ? 16 / sizeof(T) : 1;
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
        T v[VEC];
        if constexpr (VECTOR) {     // line_len % VEC == 0: a vector is entirely inside or outside
            if (i0 < line_len) {
                const VI x = load_nt((const VI*)(in + base + i0));
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[j] = (T)x[j];
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[j] = ident;
            }
        } else {
            v[0] = i0 < line_len ? (T)in[base + i0] : ident;
        }
#pragma unroll
        for (int j = 1; j < VEC; ++j) v[j] = op(v[j - 1], v[j]);
        const T inc = wave_scan_inclusive(v[VEC - 1], op, ident);
        const T off = op(carry, wave_shift_right(inc, ident));
        carry = op(carry, read_lane(inc, WAVE - 1));
        if (i0 < line_len) {
            if constexpr (VECTOR) {
                VT o;
                if (inclusive) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) o[j] = op(off, v[j]);
                } else {
                    o[0] = off;
#pragma unroll
                    for (int j = 1; j < VEC; ++j) o[j] = op(off, v[j - 1]);
                }
                store_nt((VT*)(out + base + i0), o);
            } else {
                out[base + i0] = inclusive ? op(off, v[0]) : off;
            }
        }
    }
}

// ---- one lane per line (tiny lines, or narrow `inner`) ---------------------------------------------
template <typename In, typename T, typename Op, int BLOCK>
__global__ __launch_bounds__(BLOCK) void scan_thread_kernel(const In* __restrict__ in, T* __restrict__ out, ScanGeom g, T init,
                                                            int inclusive, Op op) {
    const int64_t line = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (line >= g.inner * g.outer) return;
    const int64_t o = line / g.inner, i = line - o * g.inner;
    const int64_t base = i + o * g.inner * g.mid;
    T acc = init;
    for (int64_t m = 0; m < g.mid; ++m) {
        const T x = (T)in[base + m * g.inner];
        if (inclusive) { acc = op(acc, x); out[base + m * g.inner] = acc; }
        else { out[base + m * g.inner] = acc; acc = op(acc, x); }
    }
}

// ---- inner >= 64: lanes along `inner`, 4 waves share the rows of a chunk -----------------------------
// grid (strips, outer).  A wave keeps R consecutive rows of its 64 * VEC columns in registers, scans
// them downwards, and the four waves exchange their column totals through LDS.
template <typename In, typename T, typename Op, bool VECTOR, int R>
__global__ __launch_bounds__(256) void scan_strided_kernel(const In* __restrict__ in, T* __restrict__ out, ScanGeom g, T init,
                                                           int inclusive, Op op) {
    constexpr int VEC = VECTOR ? 16 / sizeof(T) : 1;
    constexpr int COLS = WAVE * VEC;
    constexpr int NW = 4;
    typedef typename VecOf<T, VEC>::type VT;
    typedef typename VecOf<In, VEC>::type VI;
    __shared__ T lds[NW][COLS];
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int64_t col0 = (int64_t)blockIdx.x * COLS + (int64_t)lane * VEC;
    const bool live = col0 < g.inner;
    const int64_t slab = (int64_t)blockIdx.y * g.inner * g.mid;
    const T ident = Op::template identity<T>();
    T carry[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) carry[j] = init;
    for (int64_t m0 = 0; m0 < g.mid; m0 += NW * R) {
        const int64_t row0 = m0 + (int64_t)wave * R;
        T v[R][VEC];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (live && row0 + r < g.mid) {
                const VI x = load_nt((const VI*)(in + slab + (row0 + r) * g.inner + col0));
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
            if (live && row0 + r < g.mid) {
                VT o;
                if constexpr (VEC == 1) o = inclusive ? op(pre[0], v[r][0]) : (r == 0 ? pre[0] : op(pre[0], v[r - 1][0]));
                else {
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        o[j] = inclusive ? op(pre[j], v[r][j]) : (r == 0 ? pre[j] : op(pre[j], v[r - 1][j]));
                }
                store_nt((VT*)(out + slab + (row0 + r) * g.inner + col0), o);
            }
        }
    }
}

// ---- host side ---------------------------------------------------------------------------------------
template <typename T> struct ScanTile {            // geometry of scan_lookback_kernel<..., 256, 4>
    static constexpr int K = 4;
    static constexpr int VEC = 16 / sizeof(T);
    static constexpr int TILE = 4 * WAVE * VEC * K;  // 4096 elements of 4 bytes, 2048 of 8 bytes
};

struct ScanArgs {
    int op;
    const void* in; void* out;
    int ndim; const int64_t* shape; int dim; int inclusive;
    const void* init;
    void* ws; size_t ws_bytes; hipStream_t stream;
};

template <typename In, typename T, typename Op>
inline int32_t launch_scan(const ScanArgs& a) {
    const Op op;
    const T init = a.init ? *(const T*)a.init : Op::template identity<T>();
    const In* in = (const In*)a.in;
    T* out = (T*)a.out;
    const uint32_t mask = (a.dim >= 1 && a.dim <= a.ndim) ? (1u << (a.dim - 1)) : 0u;
    const Shape3 s = collapse3(a.ndim, a.shape, mask);
    if (s.total == 0) return RK_SUCCESS;
    ScanGeom g{s.inner, s.mid, s.outer};
    constexpr int VEC = 16 / sizeof(T);
    const bool aligned = is_aligned(in, VEC * sizeof(In)) && is_aligned(out, 16);
    const int inclusive = a.inclusive ? 1 : 0;

    if (s.inner >= 64) {
        const bool vec = aligned && (s.inner % VEC == 0);
        const int cols = WAVE * (vec ? VEC : 1);
        const int64_t strips = (s.inner + cols - 1) / cols;
        if (strips > 0x7fffffff || s.outer > 65535) return RK_ERR_TOO_LARGE;
        dim3 grid((unsigned)strips, (unsigned)s.outer);
        if (vec) scan_strided_kernel<In, T, Op, true, 8><<<grid, 256, 0, a.stream>>>(in, out, g, init, inclusive, op);
        else     scan_strided_kernel<In, T, Op, false, 8><<<grid, 256, 0, a.stream>>>(in, out, g, init, inclusive, op);
        RK_LAUNCH_CHECK();
        return RK_SUCCESS;
    }
    const int64_t nlines = s.inner * s.outer;
    if (s.inner > 1 || s.mid <= 16) {
        const int64_t blocks = (nlines + 255) / 256;
        if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
        scan_thread_kernel<In, T, Op, 256><<<(unsigned)blocks, 256, 0, a.stream>>>(in, out, g, init, inclusive, op);
        RK_LAUNCH_CHECK();
        return RK_SUCCESS;
    }
    // contiguous lines
    const bool lines_aligned = aligned && (nlines == 1 || s.mid % VEC == 0);
    if (s.mid <= 1024 && nlines >= 64) {
        const int64_t blocks = (nlines + 3) / 4;
        if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
        if (lines_aligned && s.mid % VEC == 0)
            scan_wave_lines_kernel<In, T, Op, true, 256><<<(unsigned)blocks, 256, 0, a.stream>>>(in, out, s.mid, nlines, init, inclusive, op);
        else
            scan_wave_lines_kernel<In, T, Op, false, 256><<<(unsigned)blocks, 256, 0, a.stream>>>(in, out, s.mid, nlines, init, inclusive, op);
        RK_LAUNCH_CHECK();
        return RK_SUCCESS;
    }
    constexpr int TILE = ScanTile<T>::TILE;
    const int64_t tpl = (s.mid + TILE - 1) / TILE;
    const int64_t ntiles = tpl * nlines;
    if (ntiles > 0x7fffffff) return RK_ERR_TOO_LARGE;
    if (tpl == 1) {
        if (lines_aligned)
            scan_lookback_kernel<In, T, Op, true, false, 256, 4><<<(unsigned)ntiles, 256, 0, a.stream>>>(in, out, s.mid, tpl, ntiles, init, inclusive, op, nullptr, nullptr, 0, 0);
        else
            scan_lookback_kernel<In, T, Op, false, false, 256, 4><<<(unsigned)ntiles, 256, 0, a.stream>>>(in, out, s.mid, tpl, ntiles, init, inclusive, op, nullptr, nullptr, 0, 0);
        RK_LAUNCH_CHECK();
        return RK_SUCCESS;
    }
    Workspace w{};
    const size_t need = (size_t)ntiles * Words<T>::N * sizeof(uint64_t);
    if (!carve_workspace(a.ws, a.ws_bytes, need, &w)) return RK_ERR_WORKSPACE;
    const int64_t cap = (int64_t)(w.desc_bytes / sizeof(uint64_t));
    if (lines_aligned)
        scan_lookback_kernel<In, T, Op, true, true, 256, 4><<<(unsigned)ntiles, 256, 0, a.stream>>>(in, out, s.mid, tpl, ntiles, init, inclusive, op, w.hdr, w.desc, ntiles, cap);
    else
        scan_lookback_kernel<In, T, Op, false, true, 256, 4><<<(unsigned)ntiles, 256, 0, a.stream>>>(in, out, s.mid, tpl, ntiles, init, inclusive, op, w.hdr, w.desc, ntiles, cap);
    RK_LAUNCH_CHECK();
    return RK_SUCCESS;
}

template <typename In, typename T>
inline int32_t scan_typed(const ScanArgs& a) {
    switch (a.op) {
        case RK_OP_ADD: return launch_scan<In, T, OpAdd>(a);
        case RK_OP_MUL: return launch_scan<In, T, OpMul>(a);
        case RK_OP_MAX: return launch_scan<In, T, OpMax>(a);
        case RK_OP_MIN: return launch_scan<In, T, OpMin>(a);
        default: return RK_ERR_INVALID_ARGUMENT;
    }
}

int32_t scan_f32(const ScanArgs&);
int32_t scan_f64(const ScanArgs&);
int32_t scan_i32(const ScanArgs&);
int32_t scan_i64(const ScanArgs&);
int32_t scan_u8_i64(const ScanArgs&);
int32_t scan_u8_i32(const ScanArgs&);

}  // namespace rk
