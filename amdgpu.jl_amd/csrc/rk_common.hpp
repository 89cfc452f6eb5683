// Shared host + device helpers of librk.so (gfx950 / wave64 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#include "../../include/rk.h"

// ---------------------------------------------------------------------------------------
// host helpers
// ---------------------------------------------------------------------------------------

#define RK_HIP(expr)                                      \
    do {                                                  \
        hipError_t rk_e_ = (expr);                        \
        if (rk_e_ != hipSuccess) return (int32_t)rk_e_;   \
    } while (0)

// Launch errors are per-thread state in HIP; read-and-clear right after the launch.
#define RK_LAUNCH_CHECK()                                 \
    do {                                                  \
        hipError_t rk_e_ = hipGetLastError();             \
        if (rk_e_ != hipSuccess) return (int32_t)rk_e_;   \
    } while (0)

namespace rk {

constexpr int WAVE = 64;

inline size_t dtype_size(int dt) {
    switch (dt) {
        case RK_F32: case RK_I32: case RK_U32: return 4;
        case RK_F64: case RK_I64: case RK_U64: return 8;
        case RK_U8: case RK_I8: return 1;
        case RK_F16: case RK_I16: case RK_U16: return 2;
        default: return 0;
    }
}

inline bool is_aligned(const void* p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

// Device properties the launch heuristics need; queried once per device.
struct DeviceInfo {
    int cus;        // compute units (256 on MI355X)
};
const DeviceInfo& device_info();   // rk_api.hip

// ---- workspace layout -------------------------------------------------------------------
// [0, 256)                       WsHeader
// [256, +2 MiB)                  completion tickets of the multi-workgroup reductions, one per 128-byte line
// [.., +WS_PARTIALS_BYTES)       partial results of the reductions, slice totals of the scans across rows
// [WS_DESC_OFFSET, end)          tile descriptors of the look-back scan (tagged words; kept apart
//                                from the partials so arbitrary partial bits never look like a tag)
struct WsHeader {
    uint64_t scan_counter;  // look-back scan: epoch << 32 | tile acquisitions of the running call
    uint32_t wait_failed;   // epoch of a call that gave up a bounded wait (see WaitCtl), 0 = none; read by rk_workspace_status
    uint32_t alone;         // tiles that stopped waiting and resolved their look-back alone since the workspace was prepared
    uint32_t pad[60];
};
static_assert(sizeof(WsHeader) == 256, "header is one 256-byte line");

constexpr size_t WS_HEADER_BYTES = 256;
constexpr size_t WS_TICKET_COUNT = 16384;
constexpr int TICKET_STRIDE = 32;            // uint32 slots between tickets: one 128-byte line each
constexpr int TICKET_GROUP = 32;             // workgroups that share a first-level ticket
constexpr size_t WS_TICKET_BYTES = WS_TICKET_COUNT * TICKET_STRIDE * sizeof(uint32_t);
constexpr size_t WS_PARTIALS_OFFSET = WS_HEADER_BYTES + WS_TICKET_BYTES;
constexpr size_t WS_PARTIALS_BYTES = (size_t)10 << 20;
constexpr size_t WS_DESC_OFFSET = WS_PARTIALS_OFFSET + WS_PARTIALS_BYTES;
constexpr uint32_t WS_EPOCH_FIRST = 1;

struct Workspace {
    WsHeader* hdr;
    uint32_t* tickets;
    char*     partials;
    uint64_t* desc;
    size_t    desc_bytes;
};

inline bool carve_workspace(void* ws, size_t bytes, size_t desc_needed, Workspace* out) {
    if (ws == nullptr || !is_aligned(ws, 256)) return false;
    if (bytes < WS_DESC_OFFSET + desc_needed) return false;
    out->hdr = (WsHeader*)ws;
    out->tickets = (uint32_t*)((char*)ws + WS_HEADER_BYTES);
    out->partials = (char*)ws + WS_PARTIALS_OFFSET;
    out->desc = (uint64_t*)((char*)ws + WS_DESC_OFFSET);
    out->desc_bytes = (bytes - WS_DESC_OFFSET) & ~(size_t)7;
    return true;
}

// ---- shape canonicalisation ---------------------------------------------------------------
// A column-major array with a set of marked dims collapses to alternating groups; for a
// single marked run this is (inner, mid, outer): inner = product of the unmarked dims in
// front of the run (stride 1), mid = extent of the marked run (stride inner), outer = the
// unmarked rest (stride inner * mid).
struct Shape3 {
    int64_t inner, mid, outer;
    bool    single_run;   // false: the marked dims do not form one run after dropping size-1 dims
    int64_t total;
};

inline Shape3 collapse3(int ndim, const int64_t* shape, uint32_t mask) {
    Shape3 s{1, 1, 1, true, 1};
    int state = 0;  // 0: before the run, 1: in the run, 2: after it
    for (int d = 0; d < ndim; ++d) {
        int64_t n = shape[d];
        s.total *= n;
        if (n == 1) continue;            // size-1 dims belong to whichever group is convenient
        bool marked = (mask >> d) & 1u;
        if (state == 0) {
            if (marked) { state = 1; s.mid *= n; } else s.inner *= n;
        } else if (state == 1) {
            if (marked) s.mid *= n; else { state = 2; s.outer *= n; }
        } else {
            if (marked) s.single_run = false; else s.outer *= n;
        }
    }
    return s;
}

}  // namespace rk

// ---------------------------------------------------------------------------------------
// device helpers
// ---------------------------------------------------------------------------------------
#if defined(__HIPCC__)

namespace rk {

template <typename T, int N> struct VecOf { typedef T type __attribute__((ext_vector_type(N))); };
template <typename T> struct VecOf<T, 1> { typedef T type; };

// 16-byte vectors of each element type
template <typename T> struct Vec16 {
    static constexpr int N = 16 / sizeof(T);
    typedef typename VecOf<T, N>::type type;
};

// N consecutive elements at any element-aligned address as one access: global memory takes 16-byte loads and stores
// at 4-byte alignment (only LDS wants them aligned to their size), so rows that are no whole number of vectors still
// move 16 bytes a lane (reverse of a 1001 x N Float32 array: 3.0 -> 5.9 TB/s).  For 4- and 8-byte elements.
template <typename T, int N> __device__ __forceinline__ typename VecOf<T, N>::type load_nt_elems(const T* p) {
    static_assert(sizeof(T) >= 4, "narrower elements would be split into element accesses");
    typedef T U __attribute__((ext_vector_type(N), aligned(alignof(T))));
    return __builtin_nontemporal_load((const U*)p);
}
template <typename T, int N> __device__ __forceinline__ typename VecOf<T, N>::type load_elems(const T* p) {      // cached
    static_assert(sizeof(T) >= 4, "narrower elements would be split into element accesses");
    typedef T U __attribute__((ext_vector_type(N), aligned(alignof(T))));
    return *(const U*)p;
}
template <typename T, int N> __device__ __forceinline__ void store_nt_elems(T* p, typename VecOf<T, N>::type v) {
    static_assert(sizeof(T) >= 4, "narrower elements would be split into element accesses");
    typedef T U __attribute__((ext_vector_type(N), aligned(alignof(T))));
    __builtin_nontemporal_store((U)v, (U*)p);
}

template <typename V> __device__ __forceinline__ V load_nt(const V* p) {
    return __builtin_nontemporal_load(p);
}
template <typename V> __device__ __forceinline__ void store_nt(V* p, V v) {
    __builtin_nontemporal_store(v, p);
}

// ---- cross-lane data movement on 32-bit words ---------------------------------------------
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf, bool BOUND = false>
__device__ __forceinline__ uint32_t dpp_word(uint32_t old, uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)old, (int)v, CTRL, ROW_MASK, BANK_MASK, BOUND);
}

template <typename T> struct Words {
    static constexpr int N = (sizeof(T) + 3) / 4;
    uint32_t w[N];
};
template <typename T> __device__ __forceinline__ Words<T> to_words(const T& v) {
    Words<T> r;
#pragma unroll
    for (int i = 0; i < Words<T>::N; ++i) r.w[i] = 0;
    __builtin_memcpy(&r, &v, sizeof(T));
    return r;
}
template <typename T> __device__ __forceinline__ T from_words(const Words<T>& w) {
    T v;
    __builtin_memcpy(&v, &w, sizeof(T));
    return v;
}

// DPP move of a whole value; lanes whose source is invalid or masked receive `old`.
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf, typename T>
__device__ __forceinline__ T dpp_move(const T& old, const T& v) {
    Words<T> o = to_words(old), s = to_words(v), r;
#pragma unroll
    for (int i = 0; i < Words<T>::N; ++i) r.w[i] = dpp_word<CTRL, ROW_MASK, BANK_MASK>(o.w[i], s.w[i]);
    return from_words<T>(r);
}

template <int PATTERN, typename T> __device__ __forceinline__ T swizzle_move(const T& v) {
    Words<T> s = to_words(v), r;
#pragma unroll
    for (int i = 0; i < Words<T>::N; ++i) r.w[i] = (uint32_t)__builtin_amdgcn_ds_swizzle((int)s.w[i], PATTERN);
    return from_words<T>(r);
}

template <typename T> __device__ __forceinline__ T read_lane(const T& v, int lane) {
    Words<T> s = to_words(v), r;
#pragma unroll
    for (int i = 0; i < Words<T>::N; ++i) r.w[i] = (uint32_t)__builtin_amdgcn_readlane((int)s.w[i], lane);
    return from_words<T>(r);
}

// DPP control words (GFX9 encoding)
constexpr int DPP_QUAD_XOR1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_MIRROR = 0x140;
constexpr int DPP_ROW_SHR1 = 0x111, DPP_ROW_SHR2 = 0x112, DPP_ROW_SHR4 = 0x114, DPP_ROW_SHR8 = 0x118;
constexpr int DPP_ROW_BCAST15 = 0x142, DPP_ROW_BCAST31 = 0x143;
constexpr int DPP_WAVE_SHR1 = 0x138;
constexpr int SWIZZLE_XOR16 = 0x401F;      // bit mode: and 0x1f, or 0, xor 0x10

// Reduction over the 64 lanes of a wave; the result is wave-uniform.  `op` must be
// commutative.  Four DPP butterflies inside each row of 16, one ds_swizzle across the two
// rows of a half, two v_readlane for the halves.
template <typename T, typename Op> __device__ __forceinline__ T wave_reduce(T v, Op op) {
    v = op(v, dpp_move<DPP_QUAD_XOR1>(v, v));
    v = op(v, dpp_move<DPP_QUAD_XOR2>(v, v));
    v = op(v, dpp_move<DPP_ROW_HALF_MIRROR>(v, v));
    v = op(v, dpp_move<DPP_ROW_MIRROR>(v, v));
    v = op(v, swizzle_move<SWIZZLE_XOR16>(v));
    return op(read_lane(v, 0), read_lane(v, 32));
}

// Inclusive scan over the 64 lanes of a wave (Kogge-Stone inside rows with row_shr, then
// row_bcast15 / row_bcast31 carry the row totals).  `ident` is op's neutral element.
template <typename T, typename Op> __device__ __forceinline__ T wave_scan_inclusive(T v, Op op, T ident) {
    v = op(dpp_move<DPP_ROW_SHR1>(ident, v), v);
    v = op(dpp_move<DPP_ROW_SHR2>(ident, v), v);
    v = op(dpp_move<DPP_ROW_SHR4>(ident, v), v);
    v = op(dpp_move<DPP_ROW_SHR8>(ident, v), v);
    v = op(dpp_move<DPP_ROW_BCAST15, 0xa>(ident, v), v);
    v = op(dpp_move<DPP_ROW_BCAST31, 0xc>(ident, v), v);
    return v;
}

// Value of the previous lane (lane 0 receives `ident`): turns an inclusive wave scan into
// an exclusive one without subtracting.
template <typename T> __device__ __forceinline__ T wave_shift_right(T v, T ident) {
    return dpp_move<DPP_WAVE_SHR1>(ident, v);
}

__device__ __forceinline__ int lane_id() { return (int)__lane_id(); }

// ---- hand-off of small values between workgroups ---------------------------------------------
// Values are written and read word by word with relaxed agent-scope atomics: such accesses are
// performed at the device-coherent level and need no cache write-back or invalidate.  A full
// release fence at agent scope writes back the whole L2 of the XCD; issued by thousands of
// workgroups it costs more than the streaming kernel it sits in.  The writer orders
// "value, then flag/ticket" with publish_barrier() (waits until its own stores have completed).
template <typename T> __device__ __forceinline__ void store_agent(T* p, const T& v) {
    static_assert(sizeof(T) % 4 == 0 || sizeof(T) == 1 || sizeof(T) == 2, "whole words, or one scalar of 1 or 2 bytes");
    if constexpr (sizeof(T) == 1) {
        __hip_atomic_store((uint8_t*)p, __builtin_bit_cast(uint8_t, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if constexpr (sizeof(T) == 2) {
        __hip_atomic_store((uint16_t*)p, __builtin_bit_cast(uint16_t, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if constexpr (sizeof(T) % 8 == 0 && alignof(T) >= 8) {
        uint64_t w[sizeof(T) / 8];
        __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
        for (unsigned i = 0; i < sizeof(T) / 8; ++i)
            __hip_atomic_store((uint64_t*)p + i, w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        uint32_t w[sizeof(T) / 4];
        __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
        for (unsigned i = 0; i < sizeof(T) / 4; ++i)
            __hip_atomic_store((uint32_t*)p + i, w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}
template <typename T> __device__ __forceinline__ T load_agent(const T* p) {
    static_assert(sizeof(T) % 4 == 0 || sizeof(T) == 1 || sizeof(T) == 2, "whole words, or one scalar of 1 or 2 bytes");
    T v;
    if constexpr (sizeof(T) == 1) {
        return __builtin_bit_cast(T, __hip_atomic_load((const uint8_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    } else if constexpr (sizeof(T) == 2) {
        return __builtin_bit_cast(T, __hip_atomic_load((const uint16_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    } else if constexpr (sizeof(T) % 8 == 0 && alignof(T) >= 8) {
        uint64_t w[sizeof(T) / 8];
#pragma unroll
        for (unsigned i = 0; i < sizeof(T) / 8; ++i)
            w[i] = __hip_atomic_load((const uint64_t*)p + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_memcpy(&v, w, sizeof(T));
    } else {
        uint32_t w[sizeof(T) / 4];
#pragma unroll
        for (unsigned i = 0; i < sizeof(T) / 4; ++i)
            w[i] = __hip_atomic_load((const uint32_t*)p + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_memcpy(&v, w, sizeof(T));
    }
    return v;
}
// All earlier stores of this thread have completed (s_waitcnt vmcnt(0)) before anything later issues.
// ASSUMPTION beyond the HIP memory model: the model orders a relaxed store before a later relaxed atomic of the same
// thread only through a release at the scope of the reader (agent), which here would write back the L2.  What this
// relies on instead is how gfx950 executes the two: agent-scope atomic stores bypass the non-coherent caches and are
// performed at the device-coherent level, and vmcnt counts a store as done only when that level has acknowledged it,
// so a ticket or flag issued after the wait cannot be observed before the value.  The workgroup-scope fence only
// keeps the compiler from moving memory operations across this point.  True on gfx942 / gfx950; to be re-checked
// on any other target.
__device__ __forceinline__ void publish_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
}

// ---- bounded waits ------------------------------------------------------------------------------------------
// Every loop that polls memory written by another workgroup (look-back of the scans, of the select and of the
// sort) counts its unsuccessful rounds.  When one wait has used `budget` rounds -- which only happens when the
// state it polls is not what the protocol expects: a workspace that was never prepared, or one shared by calls
// that run at the same time -- it writes the call's `stamp` into the word `failed`, stops waiting and carries on
// with a meaningless value, so that every workgroup still runs to its end and the kernel exits normally.  All
// waiters of the SAME call look at `failed` every few rounds and give up with the first one; a stamp left by an
// earlier call (the word stays set until the host has read it and prepared the workspace again) is not theirs and
// does not stop them.  The results of the call that gave up are wrong; the host learns of it through
// rk_workspace_status / rk_sort_status.
struct WaitCtl {
    uint32_t* failed;
    long long budget;       // unsuccessful poll rounds one wait may spend (a round is a device-coherent load: ~1 us)
    int       backoff;      // s_sleep units between rounds
    uint32_t  stamp;        // nonzero mark of the running call: the scan epoch (set by the kernel), 1 in the sort's own control block
};
// Called once per unsuccessful round by (at least) one full wave; true = stop waiting.
__device__ __forceinline__ bool wait_give_up(const WaitCtl& w, long long& rounds) {
    ++rounds;
    if (rounds >= w.budget) {
        __hip_atomic_store(w.failed, w.stamp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return true;
    }
    if ((rounds & 31) == 0 && __hip_atomic_load(w.failed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == w.stamp) return true;
    for (int b = 0; b < w.backoff; ++b) __builtin_amdgcn_s_sleep(8);
    return false;
}

// Reduction over a workgroup of NW waves.  Every thread returns the total.  `lds` must
// hold NW values of T; safe to call repeatedly (leading barrier protects the buffer).
template <int NW, typename T, typename Op>
__device__ __forceinline__ T block_reduce(T v, Op op, T* lds) {
    v = wave_reduce(v, op);
    if constexpr (NW == 1) return v;
    const int wave = threadIdx.x / WAVE;
    __syncthreads();
    if (lane_id() == 0) lds[wave] = v;
    __syncthreads();
    T r = lds[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) r = op(r, lds[i]);
    return r;
}

// ---- element-wise maps f of mapreduce(f, op, A) ----------------------------------------------
struct MapIdentity { template <typename T> __device__ __forceinline__ T operator()(T x) const { return x; } };
struct MapAbs2     { template <typename T> __device__ __forceinline__ T operator()(T x) const { return x * x; } };
struct MapAbs {
    template <typename T> __device__ __forceinline__ T operator()(T x) const {
        if constexpr (std::is_unsigned<T>::value) return x; else return x < T(0) ? T(0) - x : x;
    }
};

// ---- reduction operators ------------------------------------------------------------------
template <typename T> struct Limits;
template <> struct Limits<float>    { static __host__ __device__ float lowest() { return -__builtin_inff(); } static __host__ __device__ float highest() { return __builtin_inff(); } };
template <> struct Limits<double>   { static __host__ __device__ double lowest() { return -__builtin_inf(); } static __host__ __device__ double highest() { return __builtin_inf(); } };
template <> struct Limits<int32_t>  { static __host__ __device__ int32_t lowest() { return INT32_MIN; } static __host__ __device__ int32_t highest() { return INT32_MAX; } };
template <> struct Limits<int64_t>  { static __host__ __device__ int64_t lowest() { return INT64_MIN; } static __host__ __device__ int64_t highest() { return INT64_MAX; } };
template <> struct Limits<uint32_t> { static __host__ __device__ uint32_t lowest() { return 0; } static __host__ __device__ uint32_t highest() { return UINT32_MAX; } };
template <> struct Limits<uint64_t> { static __host__ __device__ uint64_t lowest() { return 0; } static __host__ __device__ uint64_t highest() { return UINT64_MAX; } };
template <> struct Limits<uint8_t>  { static __host__ __device__ uint8_t lowest() { return 0; } static __host__ __device__ uint8_t highest() { return 255; } };
template <> struct Limits<int8_t>   { static __host__ __device__ int8_t lowest() { return INT8_MIN; } static __host__ __device__ int8_t highest() { return INT8_MAX; } };
template <> struct Limits<int16_t>  { static __host__ __device__ int16_t lowest() { return INT16_MIN; } static __host__ __device__ int16_t highest() { return INT16_MAX; } };
template <> struct Limits<uint16_t> { static __host__ __device__ uint16_t lowest() { return 0; } static __host__ __device__ uint16_t highest() { return UINT16_MAX; } };

// Integer arithmetic wraps like Julia's: do it on the unsigned counterpart.
template <typename T> __host__ __device__ __forceinline__ T wrap_add(T a, T b) {
    if constexpr (std::is_integral<T>::value) { typedef typename std::make_unsigned<T>::type U; return (T)((U)a + (U)b); }
    else return a + b;
}
template <typename T> __host__ __device__ __forceinline__ T wrap_mul(T a, T b) {
    if constexpr (std::is_integral<T>::value) { typedef typename std::make_unsigned<T>::type U; return (T)((U)a * (U)b); }
    else return a * b;
}

struct OpAdd {
    template <typename T> __host__ __device__ __forceinline__ T operator()(T a, T b) const { return wrap_add(a, b); }
    template <typename T> static __host__ __device__ __forceinline__ T identity() { return T(0); }
};
struct OpMul {
    template <typename T> __host__ __device__ __forceinline__ T operator()(T a, T b) const { return wrap_mul(a, b); }
    template <typename T> static __host__ __device__ __forceinline__ T identity() { return T(1); }
};
// Base.max / Base.min: NaN propagates; max(-0.0, 0.0) == 0.0, min(-0.0, 0.0) == -0.0 -- the `maximum` / `minimum` of
// IEEE 754-2019, which gfx950 has as ONE instruction (v_maximum3_f32 / v_minimum3_f32; Float64: v_max_f64 plus an
// unordered compare and selects).  Spelled out with comparisons the operator cost a dozen instructions and branches
// per element, and maximum(Float32[2^26]) ran at 46 % of the HBM peak where sum reaches 79 %.
struct OpMax {
    template <typename T> __host__ __device__ __forceinline__ T operator()(T a, T b) const {
        if constexpr (std::is_floating_point<T>::value) return __builtin_elementwise_maximum(a, b);
        else return a > b ? a : b;
    }
    template <typename T> static __host__ __device__ __forceinline__ T identity() { return Limits<T>::lowest(); }
};
struct OpMin {
    template <typename T> __host__ __device__ __forceinline__ T operator()(T a, T b) const {
        if constexpr (std::is_floating_point<T>::value) return __builtin_elementwise_minimum(a, b);
        else return a < b ? a : b;
    }
    template <typename T> static __host__ __device__ __forceinline__ T identity() { return Limits<T>::highest(); }
};

// Bitwise operators (scans of integer element types): & | xor.
struct OpAnd {
    template <typename T> __host__ __device__ __forceinline__ T operator()(T a, T b) const { return (T)(a & b); }
    template <typename T> static __host__ __device__ __forceinline__ T identity() { return (T)~(T)0; }
};
struct OpOr {
    template <typename T> __host__ __device__ __forceinline__ T operator()(T a, T b) const { return (T)(a | b); }
    template <typename T> static __host__ __device__ __forceinline__ T identity() { return T(0); }
};
struct OpXor {
    template <typename T> __host__ __device__ __forceinline__ T operator()(T a, T b) const { return (T)(a ^ b); }
    template <typename T> static __host__ __device__ __forceinline__ T identity() { return T(0); }
};

// ---- findmax / findmin: argmax over order-preserving integer keys ------------------------------
// Base.isless is a total order on floats (-0.0 < 0.0, NaN above everything) and findmax keeps the
// first maximum; findmin (Base.isgreater) keeps the first minimum but NaN still wins.  Each value
// is mapped to a signed integer key that is monotone in that order, so the reduction itself is a
// plain integer argmax with "smaller index wins ties" -- commutative and associative, hence any
// reduction tree returns what the sequential scan returns.
template <typename T> struct OrderKey;
template <> struct OrderKey<float> {
    typedef int32_t Key;
    static constexpr bool LOWEST_FREE = true;
    static __device__ __forceinline__ Key make(float v, bool want_max) {
        const int32_t b = __builtin_bit_cast(int32_t, v);
        const int32_t k = b ^ ((b >> 31) & 0x7fffffff);       // sign-magnitude -> two's complement
        return (v != v) ? INT32_MAX : (want_max ? k : ~k);
    }
    static __device__ __forceinline__ float value(Key k, bool want_max) {
        if (k == INT32_MAX) return __builtin_nanf("");
        const int32_t kk = want_max ? k : ~k;
        return __builtin_bit_cast(float, kk ^ ((kk >> 31) & 0x7fffffff));
    }
};
typedef _Float16 half_t;
template <> struct OrderKey<half_t> {             // through Float32: exact both ways
    typedef int32_t Key;
    static constexpr bool LOWEST_FREE = true;
    static __device__ __forceinline__ Key make(half_t v, bool want_max) { return OrderKey<float>::make((float)v, want_max); }
    static __device__ __forceinline__ half_t value(Key k, bool want_max) { return (half_t)OrderKey<float>::value(k, want_max); }
};
template <> struct OrderKey<double> {
    typedef int64_t Key;
    static constexpr bool LOWEST_FREE = true;
    static __device__ __forceinline__ Key make(double v, bool want_max) {
        const int64_t b = __builtin_bit_cast(int64_t, v);
        const int64_t k = b ^ ((b >> 63) & INT64_MAX);
        return (v != v) ? INT64_MAX : (want_max ? k : ~k);
    }
    static __device__ __forceinline__ double value(Key k, bool want_max) {
        if (k == INT64_MAX) return __builtin_nan("");
        const int64_t kk = want_max ? k : ~k;
        return __builtin_bit_cast(double, kk ^ ((kk >> 63) & INT64_MAX));
    }
};
template <> struct OrderKey<int32_t> {
    typedef int32_t Key;
    static constexpr bool LOWEST_FREE = false;
    static __device__ __forceinline__ Key make(int32_t v, bool want_max) { return want_max ? v : ~v; }
    static __device__ __forceinline__ int32_t value(Key k, bool want_max) { return want_max ? k : ~k; }
};
template <> struct OrderKey<int64_t> {
    typedef int64_t Key;
    static constexpr bool LOWEST_FREE = false;
    static __device__ __forceinline__ Key make(int64_t v, bool want_max) { return want_max ? v : ~v; }
    static __device__ __forceinline__ int64_t value(Key k, bool want_max) { return want_max ? k : ~k; }
};

template <> struct OrderKey<uint32_t> {
    typedef int32_t Key;
    static constexpr bool LOWEST_FREE = false;
    static __device__ __forceinline__ Key make(uint32_t v, bool want_max) { const Key k = (Key)(v ^ 0x80000000u); return want_max ? k : ~k; }
    static __device__ __forceinline__ uint32_t value(Key k, bool want_max) { return (uint32_t)(want_max ? k : ~k) ^ 0x80000000u; }
};
template <> struct OrderKey<uint64_t> {
    typedef int64_t Key;
    static constexpr bool LOWEST_FREE = false;
    static __device__ __forceinline__ Key make(uint64_t v, bool want_max) { const Key k = (Key)(v ^ 0x8000000000000000ull); return want_max ? k : ~k; }
    static __device__ __forceinline__ uint64_t value(Key k, bool want_max) { return (uint64_t)(want_max ? k : ~k) ^ 0x8000000000000000ull; }
};
// narrow integers: a 32-bit key has room below the smallest value
template <> struct OrderKey<int8_t> {
    typedef int32_t Key;
    static constexpr bool LOWEST_FREE = true;
    static __device__ __forceinline__ Key make(int8_t v, bool want_max) { return want_max ? (Key)v : ~(Key)v; }
    static __device__ __forceinline__ int8_t value(Key k, bool want_max) { return (int8_t)(want_max ? k : ~k); }
};
template <> struct OrderKey<int16_t> {
    typedef int32_t Key;
    static constexpr bool LOWEST_FREE = true;
    static __device__ __forceinline__ Key make(int16_t v, bool want_max) { return want_max ? (Key)v : ~(Key)v; }
    static __device__ __forceinline__ int16_t value(Key k, bool want_max) { return (int16_t)(want_max ? k : ~k); }
};
template <> struct OrderKey<uint16_t> {
    typedef int32_t Key;
    static constexpr bool LOWEST_FREE = true;
    static __device__ __forceinline__ Key make(uint16_t v, bool want_max) { return want_max ? (Key)v : ~(Key)v; }
    static __device__ __forceinline__ uint16_t value(Key k, bool want_max) { return (uint16_t)(want_max ? k : ~k); }
};
template <> struct OrderKey<uint8_t> {            // Bool / UInt8: findfirst(bools) is findmax's index
    typedef int32_t Key;
    static constexpr bool LOWEST_FREE = true;
    static __device__ __forceinline__ Key make(uint8_t v, bool want_max) { return want_max ? (Key)v : ~(Key)v; }
    static __device__ __forceinline__ uint8_t value(Key k, bool want_max) { return (uint8_t)(want_max ? k : ~k); }
};

// `i` is the position of the element along its line (0-based), 32-bit whenever the line is shorter than
// 2^31 so that key and position travel as one 64-bit word; -1 = nothing yet.
// LOWEST_FREE: no element maps to the lowest key (true for float keys: the smallest is that of -Inf), so
// an accumulator that starts at the lowest key takes its first element on a plain "greater than".
template <typename K, typename P, bool LOWEST_FREE> struct KeyIdx {
    K k;
    P i;
};

struct OpArgKey {
    template <typename K, typename P, bool LF>
    __host__ __device__ __forceinline__ KeyIdx<K, P, LF> operator()(KeyIdx<K, P, LF> a, KeyIdx<K, P, LF> b) const {
        if (a.i < 0) return b;
        if (b.i < 0) return a;
        if (a.k != b.k) return a.k > b.k ? a : b;
        return a.i < b.i ? a : b;
    }
    template <typename A> static __host__ __device__ __forceinline__ A identity() {
        A p;
        p.k = Limits<decltype(p.k)>::lowest();
        p.i = -1;
        return p;
    }
};

// One step of a streaming accumulation: `x` comes later in index order than everything already in
// `acc`.  Generic operators just combine; the argmax only replaces on a strictly larger key.
template <typename Op, typename A> __device__ __forceinline__ A acc_step(Op op, const A& acc, const A& x) { return op(acc, x); }
template <typename K, typename P, bool LF>
__device__ __forceinline__ KeyIdx<K, P, LF> acc_step(OpArgKey, const KeyIdx<K, P, LF>& acc, const KeyIdx<K, P, LF>& x) {
    if constexpr (LF) return x.k > acc.k ? x : acc;
    else return (acc.i < 0 || x.k > acc.k) ? x : acc;
}

}  // namespace rk
#endif  // __HIPCC__
