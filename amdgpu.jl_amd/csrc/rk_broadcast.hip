// Fused broadcast: dest .= f(args...) for a flattened Broadcasted tree.
// Replaces copyto!(dest, ::Broadcasted{<:ROCArrayStyle}) (src/broadcast.jl:3-35), i.e. GPUArrays'
// one-element-per-work-item broadcast kernel carried by src/ROCKernels.jl:107-129.
//
// One kernel skeleton, two index modes, pluggable evaluators:
//   linear   every array operand has dest's shape: one flat index, 16-byte loads and stores
//   rows     operands with extruded (size-1) dims: adjacent dims with compatible strides are merged on
//            the host, lanes run along dim 0 (stride 1 or 0 per operand), a workgroup covers TY rows
//            and decomposes the row number once per thread -- no div/mod per element
//   evaluators: fused forms for the frequent trees (no interpretation at all) and a postfix
//            interpreter for everything else (uniform control flow: every lane runs the same program;
//            the value stack lives in LDS with the top of stack cached in registers).
// Arithmetic is NOT contracted into FMAs: Julia evaluates a .* x .+ y as separate mul and add.
#include <cmath>
#include <cstring>
#include <cstdlib>

#include "rk_common.hpp"
#include "rk_interp.hpp"

#pragma clang fp contract(off)

namespace rk {

constexpr int BC_BLOCK = 256;
constexpr int BC_MAX_DEPTH = 8;
constexpr int BC_RPT = 4;            // rows per thread in rows mode

struct BcOperand {
    const void* ptr;        // nullptr: scalar
    int32_t     dtype;
    int64_t     stride0;    // element stride along merged dim 0: 0 (extruded), 1 (dense) or any other (views; scalar lanes only)
    int32_t     reused;     // has an extruded dim: elements are read many times -> cached loads, not streaming
    int32_t     row_invariant;   // every stride of dims 1.. is 0: the value depends on the dim-0 index only
    int32_t     flat_dense;      // dense over the whole merged shape: the element offset is the destination's linear index
    int64_t     stride[RK_MAX_DIMS];   // element strides of merged dims 1.. (index d-1)
    double      sf;
    int64_t     si;
};

struct BcArgs {
    int32_t   n_operands, n_tokens;
    int32_t   max_depth;               // of the value stack (entries beyond the registers live in LDS)
    int32_t   tokens[RK_MAX_PROGRAM];
    BcOperand op[RK_MAX_OPERANDS];
    int32_t   ndim;                    // merged rank (>= 1)
    int64_t   shape[RK_MAX_DIMS];      // merged dest shape
    int64_t   total;
    int64_t   nrows;                   // product of shape[1..]
    int32_t   indexed;                 // indexed mode (bc_indexed_kernel) instead of rows mode
    int32_t   tx_log2;                 // rows mode: lanes along dim 0 = 1 << tx_log2
    int64_t   nxb;                     // rows mode: workgroups along dim 0
    void*     dest;
    int32_t   dest_dtype;
    int64_t   dest_stride0;            // element strides of the destination over the merged dims (dense: 1, shape[0], ...)
    int64_t   dest_stride[RK_MAX_DIMS];
    int32_t   post;                    // fused evaluators: 0, or the token applied to the result of every operation (RK_BC_ROUND_F16)
    int32_t   vecn;                    // elements a lane on the vector path: 4, or 2 when an array has 8-byte elements (16 bytes a lane)
};

// ---- typed loads / stores --------------------------------------------------------------------------
// One element at an address that is the same in every lane of the wave (an operand extruded along dim 0 -- a row
// vector against a matrix -- when a wave's lanes share their row), from memory the kernel does not write (an operand
// with an extruded dim cannot be the destination): a scalar load.  As a vector load the same request occupies the
// texture path like a full 64-lane access, once per row and operand.
template <typename S> __device__ __forceinline__ S load_wave_uniform(const S* q) {
    const uint64_t p = (uint64_t)q;
    // (the builtin returns a signed int: without the casts the low word is sign-extended over the high one)
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)p);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(p >> 32));
    const uint64_t u = ((uint64_t)hi << 32) | (uint64_t)lo;
    typedef const S __attribute__((address_space(4))) * ConstPtr;
    return *(ConstPtr)u;
}

template <typename CT, typename S, int VEC, bool CACHED>
__device__ __forceinline__ void load_as(const void* p, int64_t off, bool contiguous, bool wave_uniform, CT (&v)[VEC]) {
    const S* q = (const S*)p + off;
    if (contiguous) {
        if constexpr (VEC == 1) v[0] = (CT)q[0];
        else {
            typedef typename VecOf<S, VEC>::type V;
            V x;
            if constexpr (CACHED) x = *(const V*)q;
            else x = load_nt((const V*)q);       // single-use data streams past the caches
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] = (CT)x[j];
        }
    } else {
        CT x;
        if constexpr (sizeof(S) >= 4) x = wave_uniform ? (CT)load_wave_uniform(q) : (CT)q[0];
        else x = (CT)q[0];
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = x;
    }
}

// HOMOG: every array operand and the destination already have the compute type -- no dispatch on the
// element type anywhere in the kernel (the common all-Float32 / all-Float64 case).
template <typename CT, int VEC, bool CACHED, bool HOMOG>
__device__ __forceinline__ void load_typed(const BcOperand& o, int64_t off, bool contiguous, bool wave_uniform, CT (&v)[VEC]) {
    if constexpr (HOMOG) { load_as<CT, CT, VEC, CACHED>(o.ptr, off, contiguous, wave_uniform, v); return; }
    switch (o.dtype) {
        case RK_F32: load_as<CT, float, VEC, CACHED>(o.ptr, off, contiguous, wave_uniform, v); break;
        case RK_F64: load_as<CT, double, VEC, CACHED>(o.ptr, off, contiguous, wave_uniform, v); break;
        case RK_I32: load_as<CT, int32_t, VEC, CACHED>(o.ptr, off, contiguous, wave_uniform, v); break;
        case RK_I64: load_as<CT, int64_t, VEC, CACHED>(o.ptr, off, contiguous, wave_uniform, v); break;
        case RK_U32: load_as<CT, uint32_t, VEC, CACHED>(o.ptr, off, contiguous, wave_uniform, v); break;
        case RK_U64: load_as<CT, uint64_t, VEC, CACHED>(o.ptr, off, contiguous, wave_uniform, v); break;
        case RK_F16: load_as<CT, half_t, VEC, CACHED>(o.ptr, off, contiguous, wave_uniform, v); break;
        case RK_I8:  load_as<CT, int8_t, VEC, CACHED>(o.ptr, off, contiguous, wave_uniform, v); break;
        case RK_I16: load_as<CT, int16_t, VEC, CACHED>(o.ptr, off, contiguous, wave_uniform, v); break;
        case RK_U16: load_as<CT, uint16_t, VEC, CACHED>(o.ptr, off, contiguous, wave_uniform, v); break;
        default:     load_as<CT, uint8_t, VEC, CACHED>(o.ptr, off, contiguous, wave_uniform, v); break;
    }
}

// MAY_REUSE: rows mode, where an extruded operand is read again and again and should stay cached; the flat
// mode reads every dense operand exactly once and always streams (one branch less per operand).
template <typename CT, int VEC, bool MAY_REUSE, bool HOMOG>
__device__ __forceinline__ void load_operand(const BcOperand& o, int64_t off, bool wave_rows, CT (&v)[VEC]) {
    if (o.ptr == nullptr) {
        const CT x = (o.dtype == RK_F32 || o.dtype == RK_F64 || o.dtype == RK_F16) ? (CT)o.sf : (CT)o.si;
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = x;
        return;
    }
    const bool contiguous = o.stride0 != 0;     // on the vector path stride0 is 0 or 1; scalar lanes carry any stride in `off`
    if (MAY_REUSE && o.reused != 0) load_typed<CT, VEC, true, HOMOG>(o, off, contiguous, wave_rows, v);
    else load_typed<CT, VEC, false, HOMOG>(o, off, contiguous, false, v);
}

template <typename CT, typename D, int VEC>
__device__ __forceinline__ void store_as(void* p, int64_t off, const CT (&v)[VEC]) {
    D* q = (D*)p + off;
    if constexpr (VEC == 1) q[0] = (D)v[0];
    else {
        typedef typename VecOf<D, VEC>::type V;
        V x;
#pragma unroll
        for (int j = 0; j < VEC; ++j) x[j] = (D)v[j];
        store_nt((V*)q, x);
    }
}

template <typename CT, int VEC, bool HOMOG>
__device__ __forceinline__ void store_dest(void* p, int dtype, int64_t off, const CT (&v)[VEC]) {
    if constexpr (HOMOG) { store_as<CT, CT, VEC>(p, off, v); return; }
    switch (dtype) {
        case RK_F32: store_as<CT, float, VEC>(p, off, v); break;
        case RK_F64: store_as<CT, double, VEC>(p, off, v); break;
        case RK_I32: store_as<CT, int32_t, VEC>(p, off, v); break;
        case RK_I64: store_as<CT, int64_t, VEC>(p, off, v); break;
        case RK_U32: store_as<CT, uint32_t, VEC>(p, off, v); break;
        case RK_U64: store_as<CT, uint64_t, VEC>(p, off, v); break;
        case RK_F16: store_as<CT, half_t, VEC>(p, off, v); break;
        case RK_I8:  store_as<CT, int8_t, VEC>(p, off, v); break;
        case RK_I16: store_as<CT, int16_t, VEC>(p, off, v); break;
        case RK_U16: store_as<CT, uint16_t, VEC>(p, off, v); break;
        default:     store_as<CT, uint8_t, VEC>(p, off, v); break;
    }
}

// ---- evaluators ---------------------------------------------------------------------------------------
// Postfix interpreter (rk_interp.hpp) over the loaded operands, one vector per run.  Two vectors (or rows) per run
// would halve the scalar branches per element, but the kernel then needs 210-250 registers and loses more to
// occupancy than it gains (sqrt(x*x+y*y)-w on 512^3: 500 -> 636 us).
template <typename CT, int VEC, int NOPS_> struct BcFetch {
    static constexpr int NOPS = NOPS_;
    const CT (&in)[RK_MAX_OPERANDS][VEC];
    template <int K> __device__ __forceinline__ void get(CT (&v)[VEC]) const {
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = in[K][j];
    }
};
template <int NOPS_, bool FULL_ = true> struct EvalInterpN {
    static constexpr int NOPS = NOPS_;             // operand slots: load what the program declares, up to this many
    static constexpr bool USES_LDS = true;
    template <typename CT, int VEC, typename A>
    static __device__ __forceinline__ void run(const A& a, const CT (&in)[RK_MAX_OPERANDS][VEC], CT (&out)[VEC], CT* lds) {
        interp_run<CT, VEC, BC_BLOCK, FULL_>(a.tokens, a.n_tokens, BcFetch<CT, VEC, NOPS_>{in}, out, lds);
    }
};
// Programs over at most 4 operands (most) run a copy with half the operand registers: in rows mode it can then keep
// the loads of all of a thread's rows in flight at the occupancy of the general one, which goes row by row and is
// bound by load latency ((A .- r) .* c .+ A on 16384^2: 1.6 TB/s).
typedef EvalInterpN<RK_MAX_OPERANDS> EvalInterp;
typedef EvalInterpN<4> EvalInterp4;
// Without pow, sin, cos and tanh -- the routines that set the interpreter's register count (89 with them: five waves a
// SIMD) -- for the programs that use none of them.
typedef EvalInterpN<4, false> EvalInterp4Light;

// Programs over Float16 arrays are Float32 programs with RK_BC_ROUND_F16 behind every operation (Julia's Float16
// arithmetic: compute in Float32, round).  The planner takes those tokens out when they follow EVERY operation
// (strip_post) and the fused evaluators round each intermediate instead, so x .+ y, a .* x .+ y and the chains of
// Float16 arrays run here and not in the interpreter, which is bound by its instructions at two bytes an element
// (x .+ y of Float16[2^26]: 172 us).  One scalar branch per operation.
template <typename CT, int VEC>
__device__ __forceinline__ void bc_post(int post, CT (&v)[VEC]) {
    if constexpr (std::is_same<CT, float>::value) {
        if (post == RK_BC_ROUND_F16) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] = (CT)(half_t)v[j];
        }
    }
}

// z = a * x + y * exp(w)            tokens: 0 1 MUL 2 3 EXP MUL ADD
struct EvalAxpbyExp {
    static constexpr int NOPS = 4;
    static constexpr bool USES_LDS = false;
    template <typename CT, int VEC, typename A>
    static __device__ __forceinline__ void run(const A& a, const CT (&in)[RK_MAX_OPERANDS][VEC], CT (&out)[VEC], CT*) {
        if (a.post != 0) {
            CT p[VEC], q[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) { p[j] = in[0][j] * in[1][j]; q[j] = exp(in[3][j]); }
            bc_post<CT, VEC>(a.post, p);
            bc_post<CT, VEC>(a.post, q);
#pragma unroll
            for (int j = 0; j < VEC; ++j) q[j] = in[2][j] * q[j];
            bc_post<CT, VEC>(a.post, q);
#pragma unroll
            for (int j = 0; j < VEC; ++j) out[j] = p[j] + q[j];
            bc_post<CT, VEC>(a.post, out);
            return;
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) out[j] = in[0][j] * in[1][j] + in[2][j] * exp(in[3][j]);
    }
};
// C = A + r * c                     tokens: 0 1 2 MUL ADD
struct EvalAddMul {
    static constexpr int NOPS = 3;
    static constexpr bool USES_LDS = false;
    template <typename CT, int VEC, typename A>
    static __device__ __forceinline__ void run(const A& a, const CT (&in)[RK_MAX_OPERANDS][VEC], CT (&out)[VEC], CT*) {
        if (a.post != 0) {
            CT p[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) p[j] = in[1][j] * in[2][j];
            bc_post<CT, VEC>(a.post, p);
#pragma unroll
            for (int j = 0; j < VEC; ++j) out[j] = in[0][j] + p[j];
            bc_post<CT, VEC>(a.post, out);
            return;
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) out[j] = in[0][j] + in[1][j] * in[2][j];
    }
};
// dest = x (copy / fill / convert)  tokens: 0
struct EvalCopy {
    static constexpr int NOPS = 1;
    static constexpr bool USES_LDS = false;
    template <typename CT, int VEC, typename A>
    static __device__ __forceinline__ void run(const A&, const CT (&in)[RK_MAX_OPERANDS][VEC], CT (&out)[VEC], CT*) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) out[j] = in[0][j];
    }
};
// dest = x op y                     tokens: 0 1 <binary>
struct EvalBinary {
    static constexpr int NOPS = 2;
    static constexpr bool USES_LDS = false;
    template <typename CT, int VEC, typename A>
    static __device__ __forceinline__ void run(const A& a, const CT (&in)[RK_MAX_OPERANDS][VEC], CT (&out)[VEC], CT*) {
        // one scalar branch on the operator, then the component loop (the other way round every element
        // would evaluate pow)
#define RK_BC_BIN2(EXPR) { _Pragma("unroll") for (int j = 0; j < VEC; ++j) { const CT x = in[0][j], y = in[1][j]; out[j] = (EXPR); } } break
        switch (a.tokens[2]) {
            case RK_BC_ADD: RK_BC_BIN2(x + y);
            case RK_BC_SUB: RK_BC_BIN2(x - y);
            case RK_BC_MUL: RK_BC_BIN2(x * y);
            case RK_BC_MAX: RK_BC_BIN2(OpMax()(x, y));
            case RK_BC_MIN: RK_BC_BIN2(OpMin()(x, y));
            case RK_BC_LT: RK_BC_BIN2(x < y ? CT(1) : CT(0));
            case RK_BC_LE: RK_BC_BIN2(x <= y ? CT(1) : CT(0));
            case RK_BC_GT: RK_BC_BIN2(x > y ? CT(1) : CT(0));
            case RK_BC_GE: RK_BC_BIN2(x >= y ? CT(1) : CT(0));
            case RK_BC_EQ: RK_BC_BIN2(x == y ? CT(1) : CT(0));
            case RK_BC_NE: RK_BC_BIN2(x != y ? CT(1) : CT(0));
            case RK_BC_AND: RK_BC_BIN2(((x != CT(0)) && (y != CT(0))) ? CT(1) : CT(0));
            case RK_BC_OR: RK_BC_BIN2(((x != CT(0)) || (y != CT(0))) ? CT(1) : CT(0));
            default:
                if constexpr (std::is_floating_point<CT>::value) {
                    if (a.tokens[2] == RK_BC_DIV) {
#pragma unroll
                        for (int j = 0; j < VEC; ++j) out[j] = in[0][j] / in[1][j];
                    } else {                        // RK_BC_POW
#pragma unroll
                        for (int j = 0; j < VEC; ++j) out[j] = pow(in[0][j], in[1][j]);
                    }
                }
                break;
        }
#undef RK_BC_BIN2
        bc_post<CT, VEC>(a.post, out);
    }
};

// dest = (u op1 v) op2 w             tokens: u v <op1> w <op2>      (x .- m) ./ s,  a .* x .+ y,  x .* x .+ y
// dest = u op1 (v op2 w)             tokens: u v w <op2> <op1>      x .+ y .* z with any arithmetic operators
// Two scalar branches and no value stack: the three-operand trees that the interpreter would run at a third to
// two thirds of the bandwidth.  The host renumbers the operands to u = 0, v = 1, w = 2 (an array that appears twice
// gets two slots): choosing among the loaded operands in the kernel, by switch or by select, makes the compiler
// index the operand registers with a computed address, i.e. move them to private memory (4x slower).
struct EvalChain2 {
    static constexpr int NOPS = 3;
    static constexpr bool USES_LDS = false;
    static bool chain_op(int t, bool int_compute) { return t >= RK_BC_ADD && t <= RK_BC_MIN && !(int_compute && t == RK_BC_DIV); }
    // true: `c` is `a` with the operands in the order u, v, w and tokens 0 1 <op1> 2 <op2> or 0 1 2 <op2> <op1>
    static bool canonical(const BcArgs& a, bool int_compute, BcArgs& c) {
        if (a.n_tokens != 5) return false;
        const int32_t* t = a.tokens;
        auto opnd = [&](int i) { return t[i] >= 0 && t[i] < a.n_operands; };
        if (!opnd(0) || !opnd(1) || !chain_op(t[4], int_compute)) return false;
        const bool left = opnd(3);                  // (u op1 v) op2 w
        if (left ? !chain_op(t[2], int_compute) : !(opnd(2) && chain_op(t[3], int_compute))) return false;
        c = a;
        c.n_operands = 3;
        c.op[0] = a.op[t[0]];
        c.op[1] = a.op[t[1]];
        c.op[2] = a.op[left ? t[3] : t[2]];
        c.tokens[0] = 0;
        c.tokens[1] = 1;
        if (left) { c.tokens[3] = 2; } else { c.tokens[2] = 2; }
        return true;
    }
    template <typename CT, int VEC>
    static __device__ __forceinline__ void apply(int tok, const CT (&x)[VEC], const CT (&y)[VEC], CT (&r)[VEC]) {
#define RK_BC_BIN3(EXPR) { _Pragma("unroll") for (int j = 0; j < VEC; ++j) { const CT p = x[j], q = y[j]; r[j] = (EXPR); } } break
        switch (tok) {
            case RK_BC_ADD: RK_BC_BIN3(p + q);
            case RK_BC_SUB: RK_BC_BIN3(p - q);
            case RK_BC_MUL: RK_BC_BIN3(p * q);
            case RK_BC_MAX: RK_BC_BIN3(OpMax()(p, q));
            case RK_BC_MIN: RK_BC_BIN3(OpMin()(p, q));
            default:
                if constexpr (std::is_floating_point<CT>::value) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) r[j] = x[j] / y[j];
                }
                break;
        }
#undef RK_BC_BIN3
    }
    template <typename CT, int VEC, typename A>
    static __device__ __forceinline__ void run(const A& a, const CT (&in)[RK_MAX_OPERANDS][VEC], CT (&out)[VEC], CT*) {
        CT t[VEC];
        if (a.tokens[3] == 2) {                     // (u op1 v) op2 w
            apply<CT, VEC>(a.tokens[2], in[0], in[1], t);
            bc_post<CT, VEC>(a.post, t);
            apply<CT, VEC>(a.tokens[4], t, in[2], out);
        } else {                                    // u op1 (v op2 w)
            apply<CT, VEC>(a.tokens[3], in[1], in[2], t);
            bc_post<CT, VEC>(a.post, t);
            apply<CT, VEC>(a.tokens[4], in[0], t, out);
        }
        bc_post<CT, VEC>(a.post, out);
    }
};

// dest = (((u0 op1 u1) op2 u2) ... opn un)      tokens: u0 u1 <op1> u2 <op2> ... un <opn>, up to 8 operands
// e.g. (x .- m) ./ s .* g .+ b.  One scalar branch per operator and no value stack; operands renumbered on the host
// to u_k = slot k, like EvalChain2.  In rows mode the interpreter is instruction-bound (1.9 TB/s on 16384^2).
// Instantiated for 4, 6 and 8 operand slots: in rows mode every slot costs scalar registers for its pointer and
// strides, and the 8-slot kernel spills some sixty of them ((A .- m) ./ s .* g .+ b with four row vectors on
// 16384^2: 2.0 TB/s with 8 slots, 2.6 with 6; a four-operand chain: 2.2 -> 3.9).  An array that appears twice is
// loaded twice.
template <int NOPS_> struct EvalLeftChainN {
    static constexpr int NOPS = NOPS_;
    static constexpr bool USES_LDS = false;
    static bool canonical(const BcArgs& a, bool int_compute, BcArgs& c) {
        const int n = (a.n_tokens + 1) / 2;         // operands of the chain
        if (a.n_tokens < 7 || a.n_tokens % 2 == 0 || n > RK_MAX_OPERANDS) return false;
        const int32_t* t = a.tokens;
        auto opnd = [&](int i) { return t[i] >= 0 && t[i] < a.n_operands; };
        if (!opnd(0)) return false;
        for (int k = 1; k < n; ++k)
            if (!opnd(2 * k - 1) || !EvalChain2::chain_op(t[2 * k], int_compute)) return false;
        c = a;
        c.n_operands = n;
        c.op[0] = a.op[t[0]];
        c.tokens[0] = 0;
        for (int k = 1; k < n; ++k) {
            c.op[k] = a.op[t[2 * k - 1]];
            c.tokens[2 * k - 1] = k;
        }
        return true;
    }
    template <typename CT, int VEC, typename A>
    static __device__ __forceinline__ void run(const A& a, const CT (&in)[RK_MAX_OPERANDS][VEC], CT (&out)[VEC], CT*) {
        CT acc[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] = in[0][j];
#pragma unroll
        for (int k = 1; k < NOPS_; ++k) {
            if (k < a.n_operands) {
                CT r[VEC];
                EvalChain2::apply<CT, VEC>(a.tokens[2 * k], acc, in[k], r);
                bc_post<CT, VEC>(a.post, r);
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[j] = r[j];
            }
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) out[j] = acc[j];
    }
};

// dest = g2(g1(f0b(f0a(u)) op f1b(f1a(v))))  or  g2(g1(f0b(f0a(u))))
// One or two operands with up to two unary functions each, a binary operator, up to two unary functions of the result:
// exp.(x), -x, sqrt.(abs.(x)), x .* x, abs2.(x) .+ abs2.(y), 1 ./ (1 .+ exp.(.-x)), abs2.(x .- y).  The host parses the
// postfix program into this shape (tree2_canonical) and passes seven codes in place of the tokens -- 0 = nothing -- so
// the kernel runs a fixed sequence of scalar branches and keeps no value stack: the interpreter moves its four register
// slots on every push and pop, some 200 instructions a vector for -x, which is what bounds it once an element has
// two bytes (-x of Float16[2^26]: 76 us, as long as for Float32).  v == u: one load (the host leaves one operand and
// sets the eighth code).  FULL = false leaves out pow, sin, cos, tanh, whose routines set the register count.
// A "unary function" may also be a binary operator with a scalar: c op t or t op c (1 ./ t, 1 .+ t, a .* x): up to two
// such scalars travel as operands 2 and 3, and the code of the slot says which and on which side
// (token | (operand + 1) << 8 | scalar_on_the_left << 16).  So a .* x .+ b .* y and 1 ./ (1 .+ exp.(.-x)) are trees of
// this form as well.
enum { T2_F0A = 0, T2_F0B, T2_F1A, T2_F1B, T2_OP, T2_G1, T2_G2, T2_SAME, T2_CODES };
template <bool FULL, int NOPS_> struct EvalTree2T {        // NOPS_ = 2: no scalar slots
    static constexpr int NOPS = NOPS_;
    static constexpr bool USES_LDS = false;
    template <typename CT, int VEC>
    static __device__ __forceinline__ void unary(int tok, int post, CT (&v)[VEC]) {
        if (tok == 0) return;
#define RK_T2_UN(EXPR) { _Pragma("unroll") for (int j = 0; j < VEC; ++j) { const CT x = v[j]; v[j] = (EXPR); } } break
        switch (tok) {
            case RK_BC_NEG: RK_T2_UN(-x);
            case RK_BC_ABS: RK_T2_UN(x < CT(0) ? -x : (x == CT(0) ? CT(0) : x));
            case RK_BC_ABS2: RK_T2_UN(x * x);
            case RK_BC_NOT: RK_T2_UN(x == CT(0) ? CT(1) : CT(0));
            default:
                if constexpr (std::is_floating_point<CT>::value) {
                    switch (tok) {
                        case RK_BC_SQRT: RK_T2_UN(sqrt(x));
                        case RK_BC_EXP: RK_T2_UN(exp(x));
                        case RK_BC_LOG: RK_T2_UN(log(x));
                        case RK_BC_INV: RK_T2_UN(CT(1) / x);
                        case RK_BC_ISNAN: RK_T2_UN(x != x ? CT(1) : CT(0));
                        case RK_BC_ROUND_F16: RK_T2_UN((CT)(half_t)x);      // a program that rounds in some places only
                        default:
                            if constexpr (FULL) {
                                switch (tok) {
                                    case RK_BC_SIN: RK_T2_UN(sin(x));
                                    case RK_BC_COS: RK_T2_UN(cos(x));
                                    case RK_BC_TANH: RK_T2_UN(tanh(x));
                                    default: break;
                                }
                            }
                            break;
                    }
                } else {
                    switch (tok) {
                        case RK_BC_ISODD: RK_T2_UN(x & CT(1));
                        case RK_BC_ISEVEN: RK_T2_UN((x & CT(1)) ^ CT(1));
                        case RK_BC_ISNAN: RK_T2_UN(x * CT(0));
                        case RK_BC_WRAP_I32: RK_T2_UN((CT)(int32_t)x);
                        case RK_BC_WRAP_U32: RK_T2_UN((CT)(uint32_t)x);
                        case RK_BC_WRAP_I8: RK_T2_UN((CT)(int8_t)x);
                        case RK_BC_WRAP_U8: RK_T2_UN((CT)(uint8_t)x);
                        case RK_BC_WRAP_I16: RK_T2_UN((CT)(int16_t)x);
                        case RK_BC_WRAP_U16: RK_T2_UN((CT)(uint16_t)x);
                        default: break;
                    }
                }
                break;
        }
#undef RK_T2_UN
        bc_post<CT, VEC>(post, v);
    }
    template <typename CT, int VEC>
    static __device__ __forceinline__ void binary(int tok, CT (&x)[VEC], const CT (&y)[VEC]) {
#define RK_T2_BIN(EXPR) { _Pragma("unroll") for (int j = 0; j < VEC; ++j) { const CT p = x[j], q = y[j]; x[j] = (EXPR); } } break
        switch (tok) {
            case RK_BC_ADD: RK_T2_BIN(p + q);
            case RK_BC_SUB: RK_T2_BIN(p - q);
            case RK_BC_MUL: RK_T2_BIN(p * q);
            case RK_BC_MAX: RK_T2_BIN(OpMax()(p, q));
            case RK_BC_MIN: RK_T2_BIN(OpMin()(p, q));
            case RK_BC_LT: RK_T2_BIN(p < q ? CT(1) : CT(0));
            case RK_BC_LE: RK_T2_BIN(p <= q ? CT(1) : CT(0));
            case RK_BC_GT: RK_T2_BIN(p > q ? CT(1) : CT(0));
            case RK_BC_GE: RK_T2_BIN(p >= q ? CT(1) : CT(0));
            case RK_BC_EQ: RK_T2_BIN(p == q ? CT(1) : CT(0));
            case RK_BC_NE: RK_T2_BIN(p != q ? CT(1) : CT(0));
            case RK_BC_AND: RK_T2_BIN(((p != CT(0)) && (q != CT(0))) ? CT(1) : CT(0));
            case RK_BC_OR: RK_T2_BIN(((p != CT(0)) || (q != CT(0))) ? CT(1) : CT(0));
            default:
                if constexpr (std::is_floating_point<CT>::value) {
                    if (tok == RK_BC_DIV) {
#pragma unroll
                        for (int j = 0; j < VEC; ++j) x[j] = x[j] / y[j];
                    } else if constexpr (FULL) {       // RK_BC_POW
#pragma unroll
                        for (int j = 0; j < VEC; ++j) x[j] = pow(x[j], y[j]);
                    }
                }
                break;
        }
#undef RK_T2_BIN
    }
    template <typename CT, int VEC, typename A>
    static __device__ __forceinline__ void run(const A& a, const CT (&in)[RK_MAX_OPERANDS][VEC], CT (&out)[VEC], CT*) {
        // one slot: a unary function, or a binary operator with the scalar in operand 2 or 3
        auto slot = [&](int code, CT (&v)[VEC]) {
            const int k = (code >> 8) & 0xff;
            if (NOPS_ < 4 || k == 0) { unary<CT, VEC>(code, a.post, v); return; }
            if constexpr (NOPS_ >= 4) {
                CT c[VEC];
#pragma unroll
                for (int j = 0; j < VEC; ++j) c[j] = k == 3 ? in[2][0] : in[3][0];      // a scalar: every component holds it
                if ((code >> 16) != 0) {            // c op v
                    binary<CT, VEC>(code & 0xff, c, v);
#pragma unroll
                    for (int j = 0; j < VEC; ++j) v[j] = c[j];
                } else {
                    binary<CT, VEC>(code & 0xff, v, c);
                }
                bc_post<CT, VEC>(a.post, v);
            }
        };
        CT x[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) x[j] = in[0][j];
        slot(a.tokens[T2_F0A], x);
        slot(a.tokens[T2_F0B], x);
        if (a.tokens[T2_OP] != 0) {
            CT y[VEC];
            if (a.tokens[T2_SAME] != 0) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) y[j] = in[0][j];
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) y[j] = in[1][j];
            }
            slot(a.tokens[T2_F1A], y);
            slot(a.tokens[T2_F1B], y);
            binary<CT, VEC>(a.tokens[T2_OP], x, y);
            bc_post<CT, VEC>(a.post, x);
        }
        slot(a.tokens[T2_G1], x);
        slot(a.tokens[T2_G2], x);
#pragma unroll
        for (int j = 0; j < VEC; ++j) out[j] = x[j];
    }
    // true: `c` is `a` in this evaluator's form; `full`: the program needs pow, sin, cos or tanh
    static bool canonical(const BcArgs& a, BcArgs& c, bool& full) {
        struct Node { int kind, tok, l, r; };        // kind 0: operand `tok`; 1: unary of l; 2: binary of l, r
        Node nodes[RK_MAX_PROGRAM];
        int stack[RK_MAX_PROGRAM], sp = 0, nn = 0;
        full = false;
        for (int i = 0; i < a.n_tokens; ++i) {
            const int tok = a.tokens[i];
            if (tok >= 0 && tok < RK_MAX_OPERANDS) { nodes[nn] = Node{0, tok, -1, -1}; stack[sp++] = nn++; continue; }
            const int ar = token_arity(tok);
            if (tok == RK_BC_IDENTITY) continue;
            if (!token_basic(tok)) full = true;
            if (ar == 1 && sp >= 1) { nodes[nn] = Node{1, tok, stack[sp - 1], -1}; stack[sp - 1] = nn++; }
            else if (ar == 2 && sp >= 2) { nodes[nn] = Node{2, tok, stack[sp - 2], stack[sp - 1]}; sp -= 1; stack[sp - 1] = nn++; }
            else return false;                      // muladd, ifelse: the interpreter's
        }
        if (sp != 1) return false;
        // unary functions -- and binary operators with a scalar -- from `n` down to the first node that is neither:
        // innermost first in f[] (as slot codes); returns that node
        int scalars[2], nscalars = 0;               // operands of `a` that travel as operands 2 and 3
        auto is_scalar = [&](int n) { return nodes[n].kind == 0 && a.op[nodes[n].tok].ptr == nullptr; };
        auto peel = [&](int n, int (&f)[4], int& nf, int limit) -> int {
            int outer_first[4];
            nf = 0;
            for (;;) {
                int code, next;
                if (nodes[n].kind == 1) { code = nodes[n].tok; next = nodes[n].l; }
                else if (nodes[n].kind == 2 && (is_scalar(nodes[n].l) != is_scalar(nodes[n].r) ||
                                                (is_scalar(nodes[n].l) && is_scalar(nodes[n].r)))) {
                    const bool left = is_scalar(nodes[n].l) && !is_scalar(nodes[n].r);     // the scalar is the left argument
                    const int sc = nodes[left ? nodes[n].l : nodes[n].r].tok;
                    int k = -1;
                    for (int i = 0; i < nscalars; ++i) if (scalars[i] == sc) k = i;
                    if (k < 0) { if (nscalars == 2) return -1; scalars[nscalars] = sc; k = nscalars++; }
                    code = nodes[n].tok | ((k + 3) << 8) | ((left ? 1 : 0) << 16);
                    next = left ? nodes[n].r : nodes[n].l;
                } else break;
                if (nf == limit) return -1;
                outer_first[nf++] = code;
                n = next;
            }
            for (int i = 0; i < nf; ++i) f[i] = outer_first[nf - 1 - i];
            return n;
        };
        int32_t code[T2_CODES] = {0, 0, 0, 0, 0, 0, 0, 0};
        int g[4], ng = 0;
        const int top = peel(stack[0], g, ng, 4);
        if (top < 0) return false;
        int ia = -1, ib = -1;
        if (nodes[top].kind == 0) {                 // unary functions of one operand only: f0a f0b g1 g2 in order of application
            if (ng == 0) return false;              // a plain copy has its own evaluator
            ia = nodes[top].tok;
            const int slot[4] = {T2_F0A, T2_F0B, T2_G1, T2_G2};
            for (int i = 0; i < ng; ++i) code[slot[i]] = g[i];
        } else {
            if (ng > 2) return false;
            int f0[4], f1[4], n0 = 0, n1 = 0;
            const int la = peel(nodes[top].l, f0, n0, 2), lb = peel(nodes[top].r, f1, n1, 2);
            if (la < 0 || lb < 0 || nodes[la].kind != 0 || nodes[lb].kind != 0) return false;
            ia = nodes[la].tok; ib = nodes[lb].tok;
            code[T2_OP] = nodes[top].tok;
            if (n0 > 0) code[T2_F0A] = f0[0];
            if (n0 > 1) code[T2_F0B] = f0[1];
            if (n1 > 0) code[T2_F1A] = f1[0];
            if (n1 > 1) code[T2_F1B] = f1[1];
            if (ng > 0) code[T2_G1] = g[0];
            if (ng > 1) code[T2_G2] = g[1];
        }
        c = a;
        c.op[0] = a.op[ia];
        c.n_operands = 1;
        if (ib >= 0) {
            if (ib == ia) code[T2_SAME] = 1;
            else { c.op[1] = a.op[ib]; c.n_operands = 2; }
        }
        if (nscalars > 0) {
            if (c.n_operands == 1) c.op[1] = a.op[scalars[0]];  // slot 1 unused: a scalar costs no load
            for (int i = 0; i < nscalars; ++i) c.op[2 + i] = a.op[scalars[i]];
            c.n_operands = 2 + nscalars;
        }
        c.n_tokens = T2_CODES;
        for (int i = 0; i < T2_CODES; ++i) c.tokens[i] = code[i];
        return true;
    }
};
// dest = g2(g1( m2(m1(f(u) op1 f(v))) op2 f(w) ))  or  g2(g1( f(w) op2 m2(m1(f(u) op1 f(v))) ))
// The same with a third operand: every f, m, g up to two unary functions or scalar operators (three distinct scalars,
// operands 3..5).  x .* y .+ sin.(w), a .* x .+ b .* y .+ c .* z, (x .- m) ./ sqrt.(v .+ eps), abs2.(x) .+ abs2.(y) .+ abs2.(z).
// Operands that are the same array are loaded once (T3_SAME_V: v is u; T3_SAME_W: 1 = w is u, 2 = w is v).
enum { T3_FU = 0, T3_FV = 2, T3_FW = 4, T3_M = 6, T3_G = 8, T3_OP1 = 10, T3_OP2, T3_W_LEFT, T3_SAME_V, T3_SAME_W, T3_CODES };
template <bool FULL> struct EvalTree3T {
    static constexpr int NOPS = 6;
    static constexpr bool USES_LDS = false;
    // flat mode only: in rows mode the compiler kept the six operand slots of several rows in private memory, and every
    // further kernel of this size costs build time
    static constexpr bool FLAT_ONLY = true;
    typedef EvalTree2T<FULL, 4> Base;
    template <typename CT, int VEC, typename A>
    static __device__ __forceinline__ void run(const A& a, const CT (&in)[RK_MAX_OPERANDS][VEC], CT (&out)[VEC], CT*) {
        auto slot = [&](int code, CT (&v)[VEC]) {
            const int k = (code >> 8) & 0xff;
            if (k == 0) { Base::template unary<CT, VEC>(code, a.post, v); return; }
            CT c[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) c[j] = k == 4 ? in[3][0] : (k == 5 ? in[4][0] : in[5][0]);
            if ((code >> 16) != 0) {            // c op v
                Base::template binary<CT, VEC>(code & 0xff, c, v);
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[j] = c[j];
            } else {
                Base::template binary<CT, VEC>(code & 0xff, v, c);
            }
            bc_post<CT, VEC>(a.post, v);
        };
        CT x[VEC], y[VEC], z[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            x[j] = in[0][j];
            y[j] = a.tokens[T3_SAME_V] != 0 ? in[0][j] : in[1][j];
            z[j] = a.tokens[T3_SAME_W] == 1 ? in[0][j] : (a.tokens[T3_SAME_W] == 2 ? in[1][j] : in[2][j]);
        }
        slot(a.tokens[T3_FU], x); slot(a.tokens[T3_FU + 1], x);
        slot(a.tokens[T3_FV], y); slot(a.tokens[T3_FV + 1], y);
        Base::template binary<CT, VEC>(a.tokens[T3_OP1], x, y);
        bc_post<CT, VEC>(a.post, x);
        slot(a.tokens[T3_M], x); slot(a.tokens[T3_M + 1], x);
        slot(a.tokens[T3_FW], z); slot(a.tokens[T3_FW + 1], z);
        if (a.tokens[T3_W_LEFT] != 0) {
            Base::template binary<CT, VEC>(a.tokens[T3_OP2], z, x);
#pragma unroll
            for (int j = 0; j < VEC; ++j) x[j] = z[j];
        } else {
            Base::template binary<CT, VEC>(a.tokens[T3_OP2], x, z);
        }
        bc_post<CT, VEC>(a.post, x);
        slot(a.tokens[T3_G], x); slot(a.tokens[T3_G + 1], x);
#pragma unroll
        for (int j = 0; j < VEC; ++j) out[j] = x[j];
    }
    static bool canonical(const BcArgs& a, BcArgs& c, bool& full) {
        struct Node { int kind, tok, l, r; };        // kind 0: operand `tok`; 1: unary of l; 2: binary of l, r
        Node nodes[RK_MAX_PROGRAM];
        int stack[RK_MAX_PROGRAM], sp = 0, nn = 0;
        full = false;
        for (int i = 0; i < a.n_tokens; ++i) {
            const int tok = a.tokens[i];
            if (tok >= 0 && tok < RK_MAX_OPERANDS) { nodes[nn] = Node{0, tok, -1, -1}; stack[sp++] = nn++; continue; }
            const int ar = token_arity(tok);
            if (tok == RK_BC_IDENTITY) continue;
            if (!token_basic(tok)) full = true;
            if (ar == 1 && sp >= 1) { nodes[nn] = Node{1, tok, stack[sp - 1], -1}; stack[sp - 1] = nn++; }
            else if (ar == 2 && sp >= 2) { nodes[nn] = Node{2, tok, stack[sp - 2], stack[sp - 1]}; sp -= 1; stack[sp - 1] = nn++; }
            else return false;
        }
        if (sp != 1) return false;
        int scalars[3], nscalars = 0;               // operands of `a` that travel as operands 3, 4, 5
        auto is_scalar = [&](int n) { return nodes[n].kind == 0 && a.op[nodes[n].tok].ptr == nullptr; };
        // up to two unary functions / scalar operators from `n` downwards, innermost first in f[]; returns the node below
        auto peel = [&](int n, int (&f)[2], int& nf) -> int {
            int outer_first[2];
            nf = 0;
            for (;;) {
                int code, next;
                if (nodes[n].kind == 1) { code = nodes[n].tok; next = nodes[n].l; }
                else if (nodes[n].kind == 2 && (is_scalar(nodes[n].l) || is_scalar(nodes[n].r))) {
                    const bool left = is_scalar(nodes[n].l) && !is_scalar(nodes[n].r);
                    const int sc = nodes[left ? nodes[n].l : nodes[n].r].tok;
                    int k = -1;
                    for (int i = 0; i < nscalars; ++i) if (scalars[i] == sc) k = i;
                    if (k < 0) { if (nscalars == 3) return -1; scalars[nscalars] = sc; k = nscalars++; }
                    code = nodes[n].tok | ((k + 4) << 8) | ((left ? 1 : 0) << 16);
                    next = left ? nodes[n].r : nodes[n].l;
                } else break;
                if (nf == 2) return -1;
                outer_first[nf++] = code;
                n = next;
            }
            for (int i = 0; i < nf; ++i) f[i] = outer_first[nf - 1 - i];
            return n;
        };
        int32_t code[T3_CODES];
        for (int i = 0; i < T3_CODES; ++i) code[i] = 0;
        auto put = [&](int at, const int (&f)[2], int nf) { for (int i = 0; i < nf; ++i) code[at + i] = f[i]; };
        int g[2], ng = 0;
        const int top = peel(stack[0], g, ng);
        if (top < 0 || nodes[top].kind != 2) return false;
        put(T3_G, g, ng);
        // one child is f(w), the other m(f(u) op1 f(v)); the left one is tried as the inner tree first
        for (int w_left = 0; w_left < 2; ++w_left) {
            const int saved = nscalars;
            const int inner_n = w_left ? nodes[top].r : nodes[top].l, leaf_n = w_left ? nodes[top].l : nodes[top].r;
            int m[2], fw[2], fu[2], fv[2], nm = 0, nw = 0, nu = 0, nv = 0;
            const int inner = peel(inner_n, m, nm);
            const int wl = peel(leaf_n, fw, nw);
            if (inner >= 0 && wl >= 0 && nodes[inner].kind == 2 && nodes[wl].kind == 0) {
                const int ul = peel(nodes[inner].l, fu, nu), vl = peel(nodes[inner].r, fv, nv);
                if (ul >= 0 && vl >= 0 && nodes[ul].kind == 0 && nodes[vl].kind == 0) {
                    const int iu = nodes[ul].tok, iv = nodes[vl].tok, iw = nodes[wl].tok;
                    for (int i = T3_FU; i < T3_G; ++i) code[i] = 0;
                    put(T3_FU, fu, nu); put(T3_FV, fv, nv); put(T3_FW, fw, nw); put(T3_M, m, nm);
                    code[T3_OP1] = nodes[inner].tok;
                    code[T3_OP2] = nodes[top].tok;
                    code[T3_W_LEFT] = w_left;
                    code[T3_SAME_V] = iv == iu ? 1 : 0;
                    code[T3_SAME_W] = iw == iu ? 1 : (iw == iv ? 2 : 0);
                    c = a;
                    const BcOperand filler = nscalars > 0 ? a.op[scalars[0]] : a.op[iu];   // unused array slots: a scalar costs no load
                    BcOperand none = filler;
                    if (nscalars == 0) { none.ptr = nullptr; none.sf = 0.0; none.si = 0; }
                    c.op[0] = a.op[iu];
                    c.op[1] = code[T3_SAME_V] ? none : a.op[iv];
                    c.op[2] = code[T3_SAME_W] ? none : a.op[iw];
                    for (int i = 0; i < 3; ++i) c.op[3 + i] = i < nscalars ? a.op[scalars[i]] : none;
                    c.n_operands = 3 + nscalars;
                    c.n_tokens = T3_CODES;
                    for (int i = 0; i < T3_CODES; ++i) c.tokens[i] = code[i];
                    return true;
                }
            }
            nscalars = saved;
        }
        return false;
    }
};
typedef EvalTree3T<false> EvalTree3Light;
typedef EvalTree3T<true> EvalTree3Full;

typedef EvalTree2T<false, 2> EvalTree2Light;
typedef EvalTree2T<true, 2> EvalTree2Full;
typedef EvalTree2T<false, 4> EvalTree2LightS;     // with scalar slots
typedef EvalTree2T<true, 4> EvalTree2FullS;

// ---- kernels --------------------------------------------------------------------------------------------
extern __shared__ __align__(16) unsigned char bc_lds_raw[];

template <typename Eval, typename CT, int VEC, bool ROWS, bool HOMOG>
__global__ __launch_bounds__(BC_BLOCK) void bc_kernel(const BcArgs a) {
    CT* lds = (CT*)bc_lds_raw;
    const int t = threadIdx.x;
    int64_t dest_off;
    int64_t off[RK_MAX_OPERANDS];
    if constexpr (!ROWS) {
        dest_off = ((int64_t)blockIdx.x * BC_BLOCK + t) * VEC;
        if (dest_off >= a.total) return;     // total % VEC == 0 on the vector path
#pragma unroll
        for (int k = 0; k < Eval::NOPS; ++k) off[k] = dest_off * a.op[k].stride0;
    } else {
        // A thread keeps its dim-0 position and takes BC_RPT rows: operands that do not depend on the row (a
        // column vector against a matrix) are loaded once.  The rows of a thread lie TY = BC_BLOCK >> tx_log2
        // apart, so that the threads of a workgroup cover TY consecutive rows with every load: with a short
        // dim 0 (4 x 32 x 262144 .+ 4 x 1 x 262144: one 16-byte vector a row) consecutive rows per thread made
        // every load touch 16 bytes in 64 (216 us; 49 us this way).
        // The fused evaluators issue the loads of all BC_RPT rows before the first use (rows past the end
        // are clamped for the loads and skipped for the store); the interpreter goes row by row.
        const int64_t xb = blockIdx.x, rb = (int64_t)blockIdx.y + (int64_t)blockIdx.z * gridDim.y;
        const int tx = t & ((1 << a.tx_log2) - 1), ty = t >> a.tx_log2;
        const int64_t i0 = ((xb << a.tx_log2) + tx) * VEC;
        const int rows_apart = BC_BLOCK >> a.tx_log2;
        const int64_t row0 = rb * (rows_apart * BC_RPT) + ty;
        if (i0 >= a.shape[0] || row0 >= a.nrows) return;
        const bool wave_rows = a.tx_log2 >= 6;     // 64 or more lanes along dim 0: the lanes of a wave share their rows
        // rows in flight per thread, bounded by registers (four operand slots of four 8-byte values each: two rows)
        constexpr int NB = Eval::USES_LDS ? (Eval::NOPS <= 4 ? 2 : 1) : ((Eval::NOPS > 4 || (Eval::NOPS > 3 && sizeof(CT) * VEC > 16)) ? 2 : BC_RPT);
        for (int r0 = 0; r0 < BC_RPT; r0 += NB) {
            CT in[NB][RK_MAX_OPERANDS][VEC];
            int64_t doff[NB];
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                int64_t row = row0 + (int64_t)(r0 + b) * rows_apart;
                if (row >= a.nrows) row = a.nrows - 1;
                // (the interpreter declares room for every operand slot: skip the 64-bit index arithmetic of the
                // slots the program does not use -- it was most of that kernel's instructions in this mode)
#pragma unroll
                for (int k = 0; k < Eval::NOPS; ++k)
                    if (!Eval::USES_LDS || k < a.n_operands) off[k] = i0 * a.op[k].stride0;
                doff[b] = i0 * a.dest_stride0;
                int64_t rem = row;
                for (int d = 1; d < a.ndim; ++d) {
                    int64_t c;
                    if (d == a.ndim - 1) c = rem;
                    else { c = rem % a.shape[d]; rem /= a.shape[d]; }
#pragma unroll
                    for (int k = 0; k < Eval::NOPS; ++k)
                        if (!Eval::USES_LDS || k < a.n_operands) off[k] += c * a.op[k].stride[d - 1];
                    doff[b] += c * a.dest_stride[d - 1];
                }
#pragma unroll
                for (int k = 0; k < Eval::NOPS; ++k) {
                    if (k >= a.n_operands) continue;
                    if (b == 0 || !a.op[k].row_invariant) load_operand<CT, VEC, true, HOMOG>(a.op[k], off[k], wave_rows, in[b][k]);
                    else {
#pragma unroll
                        for (int j = 0; j < VEC; ++j) in[b][k][j] = in[0][k][j];
                    }
                }
            }
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const int64_t row = row0 + (int64_t)(r0 + b) * rows_apart;
                if (row < a.nrows) {
                    CT out[VEC];
                    Eval::template run<CT, VEC>(a, in[b], out, lds);
                    store_dest<CT, VEC, HOMOG>(a.dest, a.dest_dtype, doff[b], out);
                }
            }
        }
        return;
    }
    // one vector per thread: two (loads of both issued first, half the workgroups) measured 4 % slower on
    // z .= a.*x .+ y.*exp.(w) and on the plain copy
    CT in[RK_MAX_OPERANDS][VEC];
#pragma unroll
    for (int k = 0; k < Eval::NOPS; ++k)
        if (k < a.n_operands) load_operand<CT, VEC, false, HOMOG>(a.op[k], off[k], false, in[k]);
    CT out[VEC];
    Eval::template run<CT, VEC>(a, in, out, lds);
    store_dest<CT, VEC, HOMOG>(a.dest, a.dest_dtype, dest_off, out);
}


// Flat mode, every array operand and the destination of the compute type, 16-byte aligned, dense (or a scalar): the
// arguments are one compact block -- all pointers side by side, scalars already in the compute type -- so a wave fetches
// them with one or two scalar loads and issues its vector loads at once.  In bc_kernel each operand's pointer, stride and
// type sit 120 bytes apart behind branches of their own: a dozen dependent scalar-load round trips in front of the
// first vector load, a fifth of the life of a wave that moves 64 bytes a lane.  Workgroups of BC_FLAT_BLOCK threads:
// the same kernel measured in one process on the same buffers at 64 / 128 / 256 / 512 / 1024 threads gave
// 6.38 / 6.41 / 6.29 / 6.24 / 6.48 TB/s at 2^26 Float32 elements, 6.38 / 6.36 / 6.18 / 6.17 / 6.34 at 2^27 and
// 6.36 / 6.25 / 6.31 / 6.24 / 6.29 at 2^28 (the plain copy: 6.70 / 6.55 / 6.51 / - / 6.41 at 2^26); two vectors a
// thread lose 1-3 % at every size, an XCD-banded order of the workgroups changes less than the run-to-run spread.
struct BcFlatArgs {
    int64_t     nvec;                       // 16-byte vectors
    void*       dest;
    const void* ptr[RK_MAX_OPERANDS];       // nullptr: scalar
    uint64_t    scalar[RK_MAX_OPERANDS];    // bits of the value in the compute type
    int32_t     n_operands, n_tokens;
    int32_t     tokens[RK_MAX_PROGRAM];
    int32_t     post;                  // always 0: the lean kernel runs homogeneous programs, which round nowhere
};
constexpr int BC_FLAT_BLOCK = 64;

// A lane moves 16 bytes: four 4-byte or two 8-byte elements.  (Four 8-byte elements a lane are two load instructions
// that each touch half of every 32 bytes of the wave's 2 KiB: copy of Float64[2^26] 278 us, 3.9 TB/s.)
template <typename Eval, typename CT, int BLOCK>
__global__ __launch_bounds__(BLOCK) void bc_flat_kernel(const BcFlatArgs a) {
    CT* lds = (CT*)bc_lds_raw;
    constexpr int FV = 16 / sizeof(CT);
    typedef typename VecOf<CT, FV>::type V;
    const int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i >= a.nvec) return;
    CT in[RK_MAX_OPERANDS][FV];
#pragma unroll
    for (int k = 0; k < Eval::NOPS; ++k) {
        if (k >= a.n_operands) continue;
        if (a.ptr[k] != nullptr) {
            const V x = load_nt((const V*)a.ptr[k] + i);
#pragma unroll
            for (int j = 0; j < FV; ++j) in[k][j] = x[j];
        } else {
            CT x;
            __builtin_memcpy(&x, &a.scalar[k], sizeof(CT));
#pragma unroll
            for (int j = 0; j < FV; ++j) in[k][j] = x;
        }
    }
    CT out[FV];
    Eval::template run<CT, FV>(a, in, out, lds);
    V o;
#pragma unroll
    for (int j = 0; j < FV; ++j) o[j] = out[j];
    store_nt((V*)a.dest + i, o);
}

static int tune_bc_narrow16() {
    const char* e = std::getenv("RK_BC_NARROW16");
    return e ? std::atoi(e) : 1;
}
static int tune_bc_flat_lean() {
    const char* e = std::getenv("RK_BC_FLAT_LEAN");
    return e ? std::atoi(e) : 1;
}

// Indexed mode: a dense destination whose rows are no whole number of 16-byte vectors (3 x N .+ 1 x N, 17 x N .* 17 x 1,
// 8191 x 4099 .+ 1 x 4099) and at most BC_INDEXED_DIMS merged dims.  Lanes along dim 0 move one element each there (and
// idle when dim 0 is short: 3 x 11184810 .+ 1 x 11184810 Float32 144 us, 63 us here); a thread owns VEC consecutive
// elements of the destination's linear order: one 16-byte store, one 16-byte load per dense operand, and for every
// other operand VEC single loads at offsets found by splitting the linear index once (three 32-bit divisions) and
// counting up with carries.
constexpr int BC_INDEXED_DIMS = 4;

template <typename Eval, typename CT, int VEC, bool HOMOG>
__global__ __launch_bounds__(BC_BLOCK) void bc_indexed_kernel(const BcArgs a) {
    CT* lds = (CT*)bc_lds_raw;
    const int64_t e0 = ((int64_t)blockIdx.x * BC_BLOCK + threadIdx.x) * VEC;
    if (e0 >= a.total) return;
    const int valid = a.total - e0 < VEC ? (int)(a.total - e0) : VEC;      // < VEC in the last thread of a ragged total
    const uint32_t s0 = (uint32_t)a.shape[0], s1 = (uint32_t)a.shape[1], s2 = (uint32_t)a.shape[2];    // 1 beyond the rank
    uint32_t c[VEC][BC_INDEXED_DIMS];
    {
        uint32_t r = (uint32_t)e0;           // total < 2^32
        c[0][0] = r % s0; r /= s0;
        c[0][1] = r % s1; r /= s1;
        c[0][2] = r % s2;
        c[0][3] = r / s2;
#pragma unroll
        for (int j = 1; j < VEC; ++j) {
            uint32_t c0 = c[j - 1][0] + 1, c1 = c[j - 1][1], c2 = c[j - 1][2], c3 = c[j - 1][3];
            if (c0 == s0) {
                c0 = 0;
                if (++c1 == s1) {
                    c1 = 0;
                    if (++c2 == s2) { c2 = 0; ++c3; }
                }
            }
            c[j][0] = c0; c[j][1] = c1; c[j][2] = c2; c[j][3] = c3;
        }
    }
    CT in[RK_MAX_OPERANDS][VEC];
#pragma unroll
    for (int k = 0; k < Eval::NOPS; ++k) {
        if (k >= a.n_operands) continue;
        const BcOperand& o = a.op[k];
        if (o.ptr == nullptr || (o.flat_dense != 0 && valid == VEC)) {
            load_operand<CT, VEC, false, HOMOG>(o, e0, false, in[k]);
        } else if (o.stride0 == 0 && s0 >= (uint32_t)(VEC - 1) && valid == VEC) {
            // extruded along dim 0 (a row vector against a matrix with short columns): the thread's VEC consecutive
            // elements cross at most one column boundary, so the first and the last offset serve all of them -- two
            // single loads instead of VEC (3 x N .+ 1 x N Float32: 61.8 -> 58.7 us)
            CT first[1], last[1];
            const int64_t off_a = (int64_t)c[0][1] * o.stride[0] + (int64_t)c[0][2] * o.stride[1] + (int64_t)c[0][3] * o.stride[2];
            const int64_t off_b = (int64_t)c[VEC - 1][1] * o.stride[0] + (int64_t)c[VEC - 1][2] * o.stride[1] + (int64_t)c[VEC - 1][3] * o.stride[2];
            load_typed<CT, 1, true, HOMOG>(o, off_a, true, false, first);
            load_typed<CT, 1, true, HOMOG>(o, off_b, true, false, last);
#pragma unroll
            for (int j = 0; j < VEC; ++j) in[k][j] = (c[0][0] + (uint32_t)j < s0) ? first[0] : last[0];
        } else if (HOMOG && sizeof(CT) >= 4 && o.stride0 == 1 && s0 >= (uint32_t)VEC && valid == VEC) {
            // contiguous along dim 0, extruded further up (a column vector against a matrix of odd height): the thread's
            // VEC elements are consecutive in the operand up to one wrap at the column's end.  Two 16-byte loads at
            // element-aligned addresses -- the column's part (starting early enough to stay inside the column) and
            // the head of the next column -- instead of VEC single ones (1001 x 60000 .+ 1001 x 1 Float32: 103 us)
            const CT* q = (const CT*)o.ptr;
            const int64_t off_a = (int64_t)c[0][1] * o.stride[0] + (int64_t)c[0][2] * o.stride[1] + (int64_t)c[0][3] * o.stride[2];
            const int64_t off_b = (int64_t)c[VEC - 1][1] * o.stride[0] + (int64_t)c[VEC - 1][2] * o.stride[1] + (int64_t)c[VEC - 1][3] * o.stride[2];
            const uint32_t start = c[0][0] + (uint32_t)VEC <= s0 ? c[0][0] : s0 - (uint32_t)VEC;
            const uint32_t d = c[0][0] - start;                         // 0 without a wrap
            const typename VecOf<CT, VEC>::type va = load_elems<CT, VEC>(q + off_a + start), vb = load_elems<CT, VEC>(q + off_b);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                CT x = va[j];
#pragma unroll
                for (int dd = 1; dd < VEC; ++dd)
                    if (d == (uint32_t)dd) x = j + dd < VEC ? va[j + dd < VEC ? j + dd : 0] : vb[j + dd >= VEC ? j + dd - VEC : 0];
                in[k][j] = x;
            }
        } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                if (j >= valid) { in[k][j] = in[k][0]; continue; }          // past the end: any value, never stored
                const int64_t off = (int64_t)c[j][0] * o.stride0 + (int64_t)c[j][1] * o.stride[0] + (int64_t)c[j][2] * o.stride[1] +
                                    (int64_t)c[j][3] * o.stride[2];
                CT one[1];
                load_typed<CT, 1, true, HOMOG>(o, off, true, false, one);
                in[k][j] = one[0];
            }
        }
    }
    CT out[VEC];
    Eval::template run<CT, VEC>(a, in, out, lds);
    if (valid == VEC) {
        store_dest<CT, VEC, HOMOG>(a.dest, a.dest_dtype, e0, out);
    } else {
#pragma unroll
        for (int j = 0; j < VEC - 1; ++j) {
            if (j >= valid) break;
            const CT one[1] = {out[j]};
            store_dest<CT, 1, HOMOG>(a.dest, a.dest_dtype, e0 + j, one);
        }
    }
}

// Eval::FLAT_ONLY = true: no rows-mode and no indexed kernels are built for the evaluator
template <typename E, typename = void> struct EvalFlatOnly : std::false_type {};
template <typename E> struct EvalFlatOnly<E, std::void_t<decltype(E::FLAT_ONLY)>> : std::integral_constant<bool, E::FLAT_ONLY> {};

template <typename Eval, typename CT>
static int32_t bc_launch(const BcArgs& a, bool vec, bool rows, hipStream_t stream) {
    const int VECN = vec ? a.vecn : 1;
    dim3 grid(1, 1, 1);
    if (!rows) {
        const int64_t blocks = (a.total / VECN + BC_BLOCK - 1) / BC_BLOCK;
        if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
        grid.x = (unsigned)blocks;
    } else {
        // x: workgroups along dim 0; (y, z): row blocks -- no division to recover them in the kernel
        const int64_t rows_per_block = (int64_t)(BC_BLOCK >> a.tx_log2) * BC_RPT;
        const int64_t row_blocks = (a.nrows + rows_per_block - 1) / rows_per_block;
        const int64_t gy = row_blocks < 32768 ? row_blocks : 32768;
        const int64_t gz = (row_blocks + gy - 1) / gy;
        if (a.nxb > 0x7fffffff || gz > 65535) return RK_ERR_TOO_LARGE;
        grid = dim3((unsigned)a.nxb, (unsigned)gy, (unsigned)gz);
    }
    // LDS only for the stack entries below the registers, i.e. for programs deeper than INTERP_REG_DEPTH
    const int spill = Eval::USES_LDS && a.max_depth > INTERP_REG_DEPTH ? a.max_depth - INTERP_REG_DEPTH : 0;
    const size_t lds = (size_t)spill * VECN * BC_BLOCK * sizeof(CT);
    // homogeneous element types: a kernel without any dispatch on the element type
    bool homog = a.dest_dtype == (std::is_same<CT, float>::value ? RK_F32 : (std::is_same<CT, double>::value ? RK_F64 : RK_I64));
    for (int k = 0; k < a.n_operands; ++k)
        if (a.op[k].ptr != nullptr && a.op[k].dtype != a.dest_dtype) homog = false;
    if (!rows && vec && homog && a.indexed == 0 && tune_bc_flat_lean() != 0) {
        // (a fill reads nothing, its workgroups live too briefly for 64 threads each: 2^26 Float32 40 -> 57 us)
        bool lean = false;
        for (int k = 0; k < a.n_operands; ++k)
            if (a.op[k].ptr != nullptr) lean = true;
        for (int k = 0; k < a.n_operands; ++k)
            if (a.op[k].ptr != nullptr && a.op[k].stride0 != 1) lean = false;      // a one-element array against a vector
        if (lean) {
            BcFlatArgs f;
            std::memset(&f, 0, sizeof(f));
            f.nvec = a.total / (16 / (int64_t)sizeof(CT));
            f.dest = a.dest;
            f.n_operands = a.n_operands;
            f.n_tokens = a.n_tokens;
            for (int i = 0; i < a.n_tokens; ++i) f.tokens[i] = a.tokens[i];
            for (int k = 0; k < a.n_operands; ++k) {
                const BcOperand& o = a.op[k];
                f.ptr[k] = o.ptr;
                if (o.ptr == nullptr) {
                    const CT x = (o.dtype == RK_F32 || o.dtype == RK_F64 || o.dtype == RK_F16) ? (CT)o.sf : (CT)o.si;
                    std::memcpy(&f.scalar[k], &x, sizeof(CT));
                }
            }
            // evaluators with a value stack in LDS index it by BC_BLOCK threads
            constexpr int FB = Eval::USES_LDS ? BC_BLOCK : BC_FLAT_BLOCK;
            const int64_t blocks = (f.nvec + FB - 1) / FB;
            if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
            bc_flat_kernel<Eval, CT, FB><<<(unsigned)blocks, FB, lds, stream>>>(f);
            RK_LAUNCH_CHECK();
            return RK_SUCCESS;
        }
    }
    // Arrays of 1- and 2-byte elements only (Float16, Int16, Bool ...): four elements a lane are 8 or 4 bytes a request,
    // too little to keep memory busy (copy of Int16[2^26] 4.9 TB/s, of Int8 3.7); eight a lane here.  The fused
    // evaluators only -- the interpreter's value stack is laid out for four.
    if constexpr (!Eval::USES_LDS) {
        if (!rows && vec && !homog && a.indexed == 0 && a.total % 8 == 0 && dtype_size((rk_dtype)a.dest_dtype) <= 2) {
            size_t widest = dtype_size((rk_dtype)a.dest_dtype);
            bool narrow = true;
            for (int k = 0; k < a.n_operands; ++k) {
                const BcOperand& o = a.op[k];
                if (o.ptr == nullptr) continue;
                if (dtype_size((rk_dtype)o.dtype) > 2) narrow = false;
                if (dtype_size((rk_dtype)o.dtype) > widest) widest = dtype_size((rk_dtype)o.dtype);
            }
            // sixteen where every array has 1-byte elements and the program is small (the operands of a lane are 16 values
            // of the compute type each)
            const int W = (widest == 1 && Eval::NOPS <= 2 && a.total % 16 == 0 && tune_bc_narrow16() != 0) ? 16 : 8;
            if (!is_aligned(a.dest, W * dtype_size((rk_dtype)a.dest_dtype))) narrow = false;
            for (int k = 0; k < a.n_operands; ++k) {
                const BcOperand& o = a.op[k];
                if (o.ptr != nullptr && o.stride0 == 1 && !is_aligned(o.ptr, W * dtype_size((rk_dtype)o.dtype))) narrow = false;
            }
            if (narrow) {
                const int64_t blocks = (a.total / W + BC_BLOCK - 1) / BC_BLOCK;
                if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
                if constexpr (Eval::NOPS <= 2) {
                    if (W == 16) {
                        bc_kernel<Eval, CT, 16, false, false><<<(unsigned)blocks, BC_BLOCK, lds, stream>>>(a);
                        RK_LAUNCH_CHECK();
                        return RK_SUCCESS;
                    }
                }
                bc_kernel<Eval, CT, 8, false, false><<<(unsigned)blocks, BC_BLOCK, lds, stream>>>(a);
                RK_LAUNCH_CHECK();
                return RK_SUCCESS;
            }
        }
    }
#define RK_BC_LAUNCH(V, R, H) bc_kernel<Eval, CT, V, R, H><<<grid, BC_BLOCK, lds, stream>>>(a)
    if constexpr (EvalFlatOnly<Eval>::value) {
        // an evaluator that exists for the flat mode only (the dispatcher sends it nothing else)
        if (rows || a.indexed != 0) return RK_ERR_UNSUPPORTED;
        if (vec && VECN == 2) { if (homog) RK_BC_LAUNCH(2, false, true); else RK_BC_LAUNCH(2, false, false); }
        else if (vec)         { if (homog) RK_BC_LAUNCH(4, false, true); else RK_BC_LAUNCH(4, false, false); }
        else                  { if (homog) RK_BC_LAUNCH(1, false, true); else RK_BC_LAUNCH(1, false, false); }
        RK_LAUNCH_CHECK();
        return RK_SUCCESS;
    } else
    if (a.indexed != 0) {            // the planner sets it together with vec and rows
        const int64_t blocks = ((a.total + VECN - 1) / VECN + BC_BLOCK - 1) / BC_BLOCK;
        if (blocks > 0x7fffffff) return RK_ERR_TOO_LARGE;
        if (VECN == 2) {
            if (homog) bc_indexed_kernel<Eval, CT, 2, true><<<(unsigned)blocks, BC_BLOCK, lds, stream>>>(a);
            else bc_indexed_kernel<Eval, CT, 2, false><<<(unsigned)blocks, BC_BLOCK, lds, stream>>>(a);
        } else if (homog) bc_indexed_kernel<Eval, CT, 4, true><<<(unsigned)blocks, BC_BLOCK, lds, stream>>>(a);
        else bc_indexed_kernel<Eval, CT, 4, false><<<(unsigned)blocks, BC_BLOCK, lds, stream>>>(a);
    } else if (vec && VECN == 2) {
        if (rows) { if (homog) RK_BC_LAUNCH(2, true, true); else RK_BC_LAUNCH(2, true, false); }
        else      { if (homog) RK_BC_LAUNCH(2, false, true); else RK_BC_LAUNCH(2, false, false); }
    } else if (vec) {
        if (rows) { if (homog) RK_BC_LAUNCH(4, true, true); else RK_BC_LAUNCH(4, true, false); }
        else      { if (homog) RK_BC_LAUNCH(4, false, true); else RK_BC_LAUNCH(4, false, false); }
    } else {
        if (rows) { if (homog) RK_BC_LAUNCH(1, true, true); else RK_BC_LAUNCH(1, true, false); }
        else      { if (homog) RK_BC_LAUNCH(1, false, true); else RK_BC_LAUNCH(1, false, false); }
    }
#undef RK_BC_LAUNCH
    RK_LAUNCH_CHECK();
    return RK_SUCCESS;
}

static bool tokens_are(const BcArgs& a, std::initializer_list<int> want) {
    if ((size_t)a.n_tokens != want.size()) return false;
    int i = 0;
    for (int w : want) if (a.tokens[i++] != w) return false;
    return true;
}

// True: `c` is `a` without its RK_BC_ROUND_F16 tokens, and c.post says that every operation rounds: the same program for
// an evaluator that rounds every intermediate (bc_post).  That holds when a rounding token follows every operation whose
// result can need one -- negation, abs, max, min, comparisons, logic and ifelse return Float16 values as they are, the
// planner need not put a token behind them, and rounding their result again changes nothing -- and behind operations only.
static bool strip_post(const BcArgs& a, BcArgs& c) {
    auto rounds = [](int tok) {
        return (tok >= RK_BC_ADD && tok <= RK_BC_DIV) || tok == RK_BC_POW || tok == RK_BC_FMA || tok == RK_BC_ABS2 ||
               (tok >= RK_BC_SQRT && tok <= RK_BC_INV);
    };
    int n = 0, posts = 0;
    int32_t t[RK_MAX_PROGRAM];
    for (int i = 0; i < a.n_tokens; ++i) {
        const int tok = a.tokens[i];
        if (tok == RK_BC_ROUND_F16) {
            if (i == 0 || a.tokens[i - 1] < RK_BC_ADD || a.tokens[i - 1] == RK_BC_ROUND_F16) return false;   // behind an operand, or twice
            ++posts;
            continue;
        }
        if (rounds(tok) && (i + 1 >= a.n_tokens || a.tokens[i + 1] != RK_BC_ROUND_F16)) return false;   // a Float32 intermediate
        t[n++] = tok;
    }
    if (posts == 0) return false;
    c = a;
    c.n_tokens = n;
    for (int i = 0; i < n; ++i) c.tokens[i] = t[i];
    c.post = RK_BC_ROUND_F16;
    return true;
}

// This file is compiled seven times: once without RK_BC_INST for the C entry points, and twice per compute type so that
// the kernel sets build in parallel -- RK_BC_INST = 0, 1, 2 (Float32, Float64, Int64): the evaluators for copies, binary
// operators and chains; RK_BC_INST = 3, 4, 5: the trees of one and two operands and the interpreters.
int32_t bc_dispatch_f32(const BcArgs& a, bool vec, bool rows, hipStream_t stream);
int32_t bc_dispatch_f64(const BcArgs& a, bool vec, bool rows, hipStream_t stream);
int32_t bc_dispatch_i64(const BcArgs& a, bool vec, bool rows, hipStream_t stream);
// second half: `only_fused` = take the program only if a fused evaluator (a tree) fits, else set taken = false
int32_t bc_rest_f32(const BcArgs& a, bool vec, bool rows, hipStream_t stream, bool only_fused, bool& taken);
int32_t bc_rest_f64(const BcArgs& a, bool vec, bool rows, hipStream_t stream, bool only_fused, bool& taken);
int32_t bc_rest_i64(const BcArgs& a, bool vec, bool rows, hipStream_t stream, bool only_fused, bool& taken);

#if defined(RK_BC_INST) && RK_BC_INST < 3
// The programs with an evaluator of their own among copies, binary operators and chains; `taken` = false: none of them.
template <typename CT>
static int32_t bc_dispatch_fused(const BcArgs& a, bool vec, bool rows, hipStream_t stream, bool& taken) {
    taken = true;
    if constexpr (std::is_floating_point<CT>::value) {
        if (tokens_are(a, {0, 1, RK_BC_MUL, 2, 3, RK_BC_EXP, RK_BC_MUL, RK_BC_ADD})) return bc_launch<EvalAxpbyExp, CT>(a, vec, rows, stream);
    }
    if (tokens_are(a, {0, 1, 2, RK_BC_MUL, RK_BC_ADD})) return bc_launch<EvalAddMul, CT>(a, vec, rows, stream);
    if (a.n_tokens == 4 && a.tokens[3] == RK_BC_FMA && a.post == 0 && a.tokens[0] >= 0 && a.tokens[0] < a.n_operands &&
        a.tokens[1] >= 0 && a.tokens[1] < a.n_operands && a.tokens[2] >= 0 && a.tokens[2] < a.n_operands) {
        // muladd.(p, q, r) = p * q + r, unfused here as in the interpreter: the same evaluator with the operands in its order
        // (not for Float16 programs: muladd rounds once, the evaluator's rounding would round the product too)
        BcArgs c = a;
        c.op[0] = a.op[a.tokens[2]];
        c.op[1] = a.op[a.tokens[0]];
        c.op[2] = a.op[a.tokens[1]];
        c.n_operands = 3;
        c.n_tokens = 5;
        const int32_t t[5] = {0, 1, 2, RK_BC_MUL, RK_BC_ADD};
        for (int i = 0; i < 5; ++i) c.tokens[i] = t[i];
        return bc_launch<EvalAddMul, CT>(c, vec, rows, stream);
    }
    if (tokens_are(a, {0})) return bc_launch<EvalCopy, CT>(a, vec, rows, stream);
    if (a.n_tokens == 3 && a.tokens[0] == 0 && a.tokens[1] == 1 &&
        ((a.tokens[2] >= RK_BC_ADD && a.tokens[2] <= RK_BC_POW && !(!std::is_floating_point<CT>::value && (a.tokens[2] == RK_BC_DIV || a.tokens[2] == RK_BC_POW))) ||
         (a.tokens[2] >= RK_BC_LT && a.tokens[2] <= RK_BC_OR)))
        return bc_launch<EvalBinary, CT>(a, vec, rows, stream);
    {
        BcArgs c;
        if (EvalChain2::canonical(a, !std::is_floating_point<CT>::value, c)) return bc_launch<EvalChain2, CT>(c, vec, rows, stream);
        if (EvalLeftChainN<8>::canonical(a, !std::is_floating_point<CT>::value, c)) {
            if (c.n_operands <= 4) return bc_launch<EvalLeftChainN<4>, CT>(c, vec, rows, stream);
            if (c.n_operands <= 6) return bc_launch<EvalLeftChainN<6>, CT>(c, vec, rows, stream);
            return bc_launch<EvalLeftChainN<8>, CT>(c, vec, rows, stream);
        }
    }
    taken = false;
    return RK_SUCCESS;
}

template <typename CT>
static int32_t bc_rest(const BcArgs& a, bool vec, bool rows, hipStream_t stream, bool only_fused, bool& taken) {
    if constexpr (std::is_same<CT, float>::value) return bc_rest_f32(a, vec, rows, stream, only_fused, taken);
    else if constexpr (std::is_same<CT, double>::value) return bc_rest_f64(a, vec, rows, stream, only_fused, taken);
    else return bc_rest_i64(a, vec, rows, stream, only_fused, taken);
}

template <typename CT>
static int32_t bc_dispatch(const BcArgs& a, bool vec, bool rows, hipStream_t stream) {
    bool taken = false;
    if constexpr (std::is_same<CT, float>::value) {
        // a Float16 program whose every operation rounds: the fused evaluators take it without the rounding tokens
        BcArgs stripped;
        if (a.post == 0 && strip_post(a, stripped)) {
            int32_t st = bc_dispatch_fused<CT>(stripped, vec, rows, stream, taken);
            if (taken) return st;
            st = bc_rest<CT>(stripped, vec, rows, stream, true, taken);
            if (taken) return st;
        }
    }
    const int32_t st = bc_dispatch_fused<CT>(a, vec, rows, stream, taken);
    if (taken) return st;
    return bc_rest<CT>(a, vec, rows, stream, false, taken);
}
#endif

#if defined(RK_BC_INST) && RK_BC_INST >= 3
template <typename CT>
static int32_t bc_rest_impl(const BcArgs& a, bool vec, bool rows, hipStream_t stream, bool only_fused, bool& taken) {
    taken = true;
    {
        BcArgs c;
        bool full = false;
        if (EvalTree2Light::canonical(a, c, full)) {
            const bool scalars = c.n_operands > 2;
            if (!full) return scalars ? bc_launch<EvalTree2LightS, CT>(c, vec, rows, stream) : bc_launch<EvalTree2Light, CT>(c, vec, rows, stream);
            // (Float64 pow / sin / cos / tanh stay with the interpreter: in rows mode the compiler kept this evaluator's
            // operands in private memory next to those routines)
            if constexpr (!std::is_same<CT, double>::value)
                return scalars ? bc_launch<EvalTree2FullS, CT>(c, vec, rows, stream) : bc_launch<EvalTree2Full, CT>(c, vec, rows, stream);
        }
    }
    {
        BcArgs c;
        bool full = false;
        if (!rows && a.indexed == 0 && EvalTree3Light::canonical(a, c, full)) {
            if (!full) return bc_launch<EvalTree3Light, CT>(c, vec, rows, stream);
            if constexpr (!std::is_same<CT, double>::value) return bc_launch<EvalTree3Full, CT>(c, vec, rows, stream);
        }
    }
    if (only_fused) { taken = false; return RK_SUCCESS; }
    if (a.n_operands <= EvalInterp4::NOPS) {
        bool heavy = false;
        for (int i = 0; i < a.n_tokens; ++i)
            if (a.tokens[i] == RK_BC_POW || a.tokens[i] == RK_BC_SIN || a.tokens[i] == RK_BC_COS || a.tokens[i] == RK_BC_TANH) heavy = true;
        if (!heavy) return bc_launch<EvalInterp4Light, CT>(a, vec, rows, stream);
        return bc_launch<EvalInterp4, CT>(a, vec, rows, stream);
    }
    return bc_launch<EvalInterp, CT>(a, vec, rows, stream);
}
#endif

#if defined(RK_BC_INST) && RK_BC_INST == 0
int32_t bc_dispatch_f32(const BcArgs& a, bool vec, bool rows, hipStream_t stream) { return bc_dispatch<float>(a, vec, rows, stream); }
#elif defined(RK_BC_INST) && RK_BC_INST == 1
int32_t bc_dispatch_f64(const BcArgs& a, bool vec, bool rows, hipStream_t stream) { return bc_dispatch<double>(a, vec, rows, stream); }
#elif defined(RK_BC_INST) && RK_BC_INST == 2
int32_t bc_dispatch_i64(const BcArgs& a, bool vec, bool rows, hipStream_t stream) { return bc_dispatch<int64_t>(a, vec, rows, stream); }
#elif defined(RK_BC_INST) && RK_BC_INST == 3
int32_t bc_rest_f32(const BcArgs& a, bool vec, bool rows, hipStream_t stream, bool only_fused, bool& taken) { return bc_rest_impl<float>(a, vec, rows, stream, only_fused, taken); }
#elif defined(RK_BC_INST) && RK_BC_INST == 4
int32_t bc_rest_f64(const BcArgs& a, bool vec, bool rows, hipStream_t stream, bool only_fused, bool& taken) { return bc_rest_impl<double>(a, vec, rows, stream, only_fused, taken); }
#elif defined(RK_BC_INST) && RK_BC_INST == 5
int32_t bc_rest_i64(const BcArgs& a, bool vec, bool rows, hipStream_t stream, bool only_fused, bool& taken) { return bc_rest_impl<int64_t>(a, vec, rows, stream, only_fused, taken); }
#endif

}  // namespace rk

#ifndef RK_BC_INST
using namespace rk;

static int32_t broadcast_impl(const rk_program* prog, void* dest, rk_dtype dest_dtype, int ndim, const int64_t* shape,
                              const int64_t* dest_strides, void* stream) {
    if (prog == nullptr) return RK_ERR_INVALID_ARGUMENT;
    if (ndim < 0 || ndim > RK_MAX_DIMS || (ndim > 0 && shape == nullptr)) return RK_ERR_INVALID_ARGUMENT;
    if ((int)dest_dtype < RK_F32 || (int)dest_dtype > RK_U16) return RK_ERR_INVALID_ARGUMENT;
    if (prog->compute != RK_F32 && prog->compute != RK_F64 && prog->compute != RK_I64) return RK_ERR_UNSUPPORTED;
    const bool int_compute = prog->compute == RK_I64;
    if (dest_dtype == RK_F16 && int_compute) return RK_ERR_UNSUPPORTED;
    if (prog->n_operands < 0 || prog->n_operands > RK_MAX_OPERANDS) return RK_ERR_INVALID_ARGUMENT;
    if (prog->n_tokens < 1 || prog->n_tokens > RK_MAX_PROGRAM) return RK_ERR_INVALID_ARGUMENT;

    int max_depth = 0;
    {
        const int32_t st = validate_tokens(prog->tokens, prog->n_tokens, prog->n_operands, int_compute, BC_MAX_DEPTH, &max_depth);
        if (st != RK_SUCCESS) return st;
    }

    int64_t total = 1;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] < 0) return RK_ERR_INVALID_ARGUMENT;
        total *= shape[d];
    }
    // operand shapes against dest (Julia: DimensionMismatch), per-dim strides with 0 on extruded dims
    // slot n_operands holds the destination, so that dims merge only where it is dense as well
    const int KD = prog->n_operands;
    int64_t stride[RK_MAX_OPERANDS + 1][RK_MAX_DIMS];
    {
        int64_t s = 1;
        for (int d = 0; d < ndim; ++d) {
            stride[KD][d] = dest_strides ? dest_strides[d] : s;
            s *= shape[d];
        }
    }
    for (int k = 0; k < prog->n_operands; ++k) {
        const rk_operand& o = prog->operands[k];
        if (o.dtype < RK_F32 || o.dtype > RK_U16) return RK_ERR_INVALID_ARGUMENT;
        if (o.dtype == RK_F16 && int_compute) return RK_ERR_UNSUPPORTED;
        if (o.ptr == nullptr) {
            if (o.ndim != 0) return RK_ERR_INVALID_ARGUMENT;
            for (int d = 0; d < ndim; ++d) stride[k][d] = 0;
            continue;
        }
        if (o.ndim < 0 || o.ndim > ndim) return o.ndim > RK_MAX_DIMS || o.ndim < 0 ? RK_ERR_INVALID_ARGUMENT : RK_ERR_DIMENSION;
        int64_t s = 1;
        for (int d = 0; d < ndim; ++d) {
            const int64_t n = d < o.ndim ? o.shape[d] : 1;
            if (n != shape[d] && n != 1) return RK_ERR_DIMENSION;
            stride[k][d] = (n == 1) ? 0 : (o.strided ? o.strides[d] : s);
            s *= n;
        }
    }
    if (total == 0) return RK_SUCCESS;
    if (dest == nullptr) return RK_ERR_INVALID_ARGUMENT;

    // merge adjacent dims: (d, d+1) merge when every operand has stride[d+1] == stride[d] * shape[d]
    // (extruded in both, or dense in both); size-1 dims vanish
    BcArgs a;
    std::memset(&a, 0, sizeof(a));
    int64_t mshape[RK_MAX_DIMS];
    int64_t mstride[RK_MAX_OPERANDS + 1][RK_MAX_DIMS];
    int m = 0;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] == 1) continue;
        bool merge = m > 0;
        if (merge)
            for (int k = 0; k <= KD; ++k)
                if (stride[k][d] != mstride[k][m - 1] * mshape[m - 1]) { merge = false; break; }
        if (merge) mshape[m - 1] *= shape[d];
        else {
            mshape[m] = shape[d];
            for (int k = 0; k <= KD; ++k) mstride[k][m] = stride[k][d];
            ++m;
        }
    }
    if (m == 0) { mshape[0] = 1; for (int k = 0; k < KD; ++k) mstride[k][0] = 0; mstride[KD][0] = 1; m = 1; }

    a.n_operands = prog->n_operands;
    a.n_tokens = prog->n_tokens;
    a.max_depth = max_depth;
    for (int i = 0; i < prog->n_tokens; ++i) a.tokens[i] = prog->tokens[i];
    a.ndim = m;
    a.total = total;
    a.nrows = 1;
    for (int d = 0; d < m; ++d) { a.shape[d] = mshape[d]; if (d > 0) a.nrows *= mshape[d]; }
    a.dest = dest;
    a.dest_dtype = (int32_t)dest_dtype;
    a.dest_stride0 = mstride[KD][0];
    for (int d = 1; d < m; ++d) a.dest_stride[d - 1] = mstride[KD][d];
    bool linear = (m == 1 && mstride[KD][0] == 1);     // the destination and every array operand dense over the merged shape
    // 16-byte lanes: whole vectors along dim 0, dense there, and every row start of every array 16-byte aligned
    bool vec = (mshape[0] % 4 == 0) && is_aligned(dest, 4 * dtype_size(dest_dtype)) && mstride[KD][0] == 1;
    for (int d = 1; d < m; ++d)
        if (mstride[KD][d] % 4 != 0) vec = false;
    for (int k = 0; k < prog->n_operands; ++k) {
        const rk_operand& o = prog->operands[k];
        BcOperand& b = a.op[k];
        b.ptr = o.ptr;
        b.dtype = o.dtype;
        b.sf = o.scalar_f;
        b.si = o.scalar_i;
        b.stride0 = mstride[k][0];
        b.row_invariant = 1;
        b.reused = (mstride[k][0] == 0) ? 1 : 0;
        for (int d = 1; d < m; ++d) {
            b.stride[d - 1] = mstride[k][d];
            if (mstride[k][d] != 0) b.row_invariant = 0;
            else b.reused = 1;
        }
        if (o.ptr != nullptr) {
            // one merged dim: the flat kernel takes operands that are dense (stride 1) or fully extruded (stride 0)
            if (mstride[k][0] != 0 && mstride[k][0] != 1) { linear = false; vec = false; }
            if (mstride[k][0] == 1) {
                if (!is_aligned(o.ptr, 4 * dtype_size(o.dtype))) vec = false;
                for (int d = 1; d < m; ++d)
                    if (mstride[k][d] % 4 != 0) vec = false;
            }
        }
    }
    if (!linear && !vec && m <= BC_INDEXED_DIMS && total < (1ll << 32) &&
        is_aligned(dest, 4 * dtype_size(dest_dtype))) {
        // rows that are no whole number of vectors, dense destination: threads along the linear index
        bool ok = mstride[KD][0] == 1;
        int64_t dense = mshape[0];
        for (int d = 1; d < m && ok; ++d) { ok = mstride[KD][d] == dense; dense *= mshape[d]; }
        for (int k = 0; k < prog->n_operands && ok; ++k) {
            if (prog->operands[k].ptr == nullptr) continue;
            bool fd = mstride[k][0] == 1;
            int64_t ds = mshape[0];
            for (int d = 1; d < m && fd; ++d) { fd = mstride[k][d] == ds; ds *= mshape[d]; }
            a.op[k].flat_dense = fd ? 1 : 0;
            if (fd && !is_aligned(prog->operands[k].ptr, 4 * dtype_size(prog->operands[k].dtype))) ok = false;
        }
        if (ok) {
            a.indexed = 1;
            vec = true;
            for (int d = m; d < BC_INDEXED_DIMS; ++d) a.shape[d] = 1;
        }
    }
    // 16 bytes a lane: two elements where an array has 8-byte elements (four would be two load instructions that each touch
    // half of every 32 bytes the wave covers: C .= A .+ r .* c on 8192^2 Float64 5.1 TB/s against 6.1 for Float32)
    a.vecn = 4;
    if (dtype_size(dest_dtype) == 8) a.vecn = 2;
    for (int k = 0; k < prog->n_operands; ++k)
        if (prog->operands[k].ptr != nullptr && dtype_size(prog->operands[k].dtype) == 8) a.vecn = 2;
    if (!linear) {
        // lanes along dim 0: TX = smallest power of two covering shape[0] / VEC, at most the workgroup
        const int vw = vec ? a.vecn : 1;
        const int64_t n0v = (mshape[0] + vw - 1) / vw;
        int l2 = 0;
        while ((1 << l2) < BC_BLOCK && (1ll << l2) < n0v) ++l2;
        a.tx_log2 = l2;
        a.nxb = (n0v + (1ll << l2) - 1) >> l2;
    }
    if (prog->compute == RK_F32) return bc_dispatch_f32(a, vec, !linear, (hipStream_t)stream);
    if (int_compute) return bc_dispatch_i64(a, vec, !linear, (hipStream_t)stream);
    return bc_dispatch_f64(a, vec, !linear, (hipStream_t)stream);
}

extern "C" int32_t rk_broadcast(const rk_program* prog, void* dest, rk_dtype dest_dtype, int ndim, const int64_t* shape,
                                void* stream) {
    return broadcast_impl(prog, dest, dest_dtype, ndim, shape, nullptr, stream);
}

extern "C" int32_t rk_broadcast_strided(const rk_program* prog, void* dest, rk_dtype dest_dtype, int ndim, const int64_t* shape,
                                        const int64_t* dest_strides, void* stream) {
    return broadcast_impl(prog, dest, dest_dtype, ndim, shape, dest_strides, stream);
}
#endif  // RK_BC_INST
