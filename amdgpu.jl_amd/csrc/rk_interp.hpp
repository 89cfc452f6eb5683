// Postfix programs (rk_bc_token): host-side validation and the device interpreter shared by the fused broadcast
// (dest .= f.(args...), src/broadcast.jl:3-35) and by reductions with a mapped element
// (mapreduce(x -> x + 1, +, A): GPUArrays.mapreducedim! with a closure for f, src/kernels/mapreduce.jl:86-89).
#pragma once
#include <type_traits>

#include "rk_common.hpp"

namespace rk {

// Number of values a token pops (it always pushes one); -1 for a token that is not an operator.
__host__ __device__ constexpr int token_arity(int tok) {
    return (tok >= RK_BC_ADD && tok <= RK_BC_POW)      ? 2
           : (tok == RK_BC_FMA)                        ? 3
           : (tok >= RK_BC_NEG && tok <= RK_BC_IDENTITY) ? 1
           : (tok >= RK_BC_LT && tok <= RK_BC_OR)      ? 2
           : (tok == RK_BC_IFELSE)                     ? 3
           : (tok >= RK_BC_NOT && tok <= RK_BC_WRAP_U16) ? 1
                                                       : -1;
}

// Tokens of the integer programs: they compute in Int64, and the store (or the WRAP tokens) keeps the low bits, so
// only operations that commute with truncation, or act on wrapped values, are allowed.
__host__ __device__ constexpr bool token_int_ok(int tok) {
    return tok == RK_BC_ADD || tok == RK_BC_SUB || tok == RK_BC_MUL || tok == RK_BC_MAX || tok == RK_BC_MIN || tok == RK_BC_FMA ||
           tok == RK_BC_NEG || tok == RK_BC_ABS || tok == RK_BC_ABS2 || tok == RK_BC_IDENTITY || (tok >= RK_BC_LT && tok <= RK_BC_OR) ||
           tok == RK_BC_IFELSE || (tok >= RK_BC_NOT && tok <= RK_BC_WRAP_U32) || (tok >= RK_BC_WRAP_I8 && tok <= RK_BC_WRAP_U16);
}
__host__ __device__ constexpr bool token_float_ok(int tok) {
    return tok != RK_BC_ISODD && tok != RK_BC_ISEVEN && tok != RK_BC_WRAP_I32 && tok != RK_BC_WRAP_U32 && !(tok >= RK_BC_WRAP_I8 && tok <= RK_BC_WRAP_U16);
}

// pow and the trigonometric / hyperbolic functions exist in the full interpreter only
__host__ __device__ constexpr bool token_basic(int tok) {
    return tok != RK_BC_POW && tok != RK_BC_SIN && tok != RK_BC_COS && tok != RK_BC_TANH;
}

// A well-formed postfix expression that leaves exactly one value; operand tokens are 0 .. n_operands-1.
inline int32_t validate_tokens(const int32_t* tokens, int n_tokens, int n_operands, bool int_compute, int max_allowed_depth,
                               int* depth_out = nullptr) {
    int depth = 0, max_depth = 0;
    for (int i = 0; i < n_tokens; ++i) {
        const int tok = tokens[i];
        if (tok >= 0 && tok < RK_MAX_OPERANDS) {
            if (tok >= n_operands) return RK_ERR_INVALID_ARGUMENT;
            ++depth;
        } else {
            const int ar = token_arity(tok);
            if (ar < 0 || depth < ar) return RK_ERR_INVALID_ARGUMENT;
            if (int_compute ? !token_int_ok(tok) : !token_float_ok(tok)) return RK_ERR_UNSUPPORTED;   // Julia: Int / Int is a Float64
            depth -= ar - 1;
        }
        if (depth > max_depth) max_depth = depth;
    }
    if (depth != 1) return RK_ERR_INVALID_ARGUMENT;
    if (max_depth > max_allowed_depth) return RK_ERR_UNSUPPORTED;
    if (depth_out) *depth_out = max_depth;
    return RK_SUCCESS;
}

// The program is the same for every lane, so every token is one scalar branch (a switch outside the per-component
// loops: inside them the compiler turns it into selects that evaluate exp, log, sin ... for every element).
// N components are evaluated together.  The four topmost stack entries live in registers and move by one place on
// push / pop; deeper entries (rare) spill to LDS when SPILL_BLOCK > 0 (entry e of thread t, component j at
// lds[(e * N + j) * SPILL_BLOCK + t]); with SPILL_BLOCK == 0 the host limits programs to depth INTERP_REG_DEPTH.
// FULL = false leaves out pow, sin, cos and tanh (the reductions instantiate the interpreter in every kernel variant;
// the host keeps such programs away from them).
// fetch.template get<K>(v) delivers operand K < Fetch::NOPS; tokens[i] is token i (an array in kernel arguments, or
// packed bits).
// Measured alternative: slots as fixed registers selected by a second switch over the (uniform) depth, so that
// nothing moves on push / pop -- more scalar branches per token and just as many moves (the register allocator
// reconciles the cases with copies): no faster, 4 MB more code.
constexpr int INTERP_REG_DEPTH = 4;

template <typename CT, int N, int SPILL_BLOCK, bool FULL, typename Tokens, typename Fetch>
__device__ __forceinline__ void interp_run(const Tokens& tokens, int n_tokens, const Fetch& fetch, CT (&out)[N], CT* lds) {
    const int t = threadIdx.x;
    CT s0[N], s1[N], s2[N], s3[N];     // s0 = top of the stack
#pragma unroll
    for (int j = 0; j < N; ++j) s0[j] = s1[j] = s2[j] = s3[j] = CT(0);
    int depth = 0;
    auto push = [&](const CT (&v)[N]) {
        if constexpr (SPILL_BLOCK > 0) {
            if (depth >= INTERP_REG_DEPTH) {
#pragma unroll
                for (int j = 0; j < N; ++j) lds[((depth - INTERP_REG_DEPTH) * N + j) * SPILL_BLOCK + t] = s3[j];
            }
        }
#pragma unroll
        for (int j = 0; j < N; ++j) { s3[j] = s2[j]; s2[j] = s1[j]; s1[j] = s0[j]; s0[j] = v[j]; }
        ++depth;
    };
    auto drop_second = [&]() {                 // the entry under the top has been consumed
        --depth;
#pragma unroll
        for (int j = 0; j < N; ++j) { s1[j] = s2[j]; s2[j] = s3[j]; }
        if constexpr (SPILL_BLOCK > 0) {
            if (depth >= INTERP_REG_DEPTH) {
#pragma unroll
                for (int j = 0; j < N; ++j) s3[j] = lds[((depth - INTERP_REG_DEPTH) * N + j) * SPILL_BLOCK + t];
            }
        }
    };
#define RK_BC_OPERAND(K) case K: { CT v[N]; if constexpr (K < Fetch::NOPS) fetch.template get<K>(v); push(v); } break
#define RK_BC_UN(EXPR)  { _Pragma("unroll") for (int j = 0; j < N; ++j) { const CT x = s0[j]; s0[j] = (EXPR); } } break
#define RK_BC_BIN(EXPR) { _Pragma("unroll") for (int j = 0; j < N; ++j) { const CT x = s1[j], y = s0[j]; s0[j] = (EXPR); } drop_second(); } break
    for (int i = 0; i < n_tokens; ++i) {
        const int tok = tokens[i];
        switch (tok) {
            RK_BC_OPERAND(0);
            RK_BC_OPERAND(1);
            RK_BC_OPERAND(2);
            RK_BC_OPERAND(3);
            RK_BC_OPERAND(4);
            RK_BC_OPERAND(5);
            RK_BC_OPERAND(6);
            RK_BC_OPERAND(7);
            case RK_BC_ADD: RK_BC_BIN(x + y);
            case RK_BC_SUB: RK_BC_BIN(x - y);
            case RK_BC_MUL: RK_BC_BIN(x * y);
            case RK_BC_MAX: RK_BC_BIN(OpMax()(x, y));
            case RK_BC_MIN: RK_BC_BIN(OpMin()(x, y));
            case RK_BC_FMA: {                   // x * y + top with x the deepest of the three
#pragma unroll
                for (int j = 0; j < N; ++j) s0[j] = s2[j] * s1[j] + s0[j];
                drop_second();
                drop_second();
            } break;
            case RK_BC_NEG: RK_BC_UN(-x);
            case RK_BC_ABS: RK_BC_UN(x < CT(0) ? -x : (x == CT(0) ? CT(0) : x));
            case RK_BC_ABS2: RK_BC_UN(x * x);
            case RK_BC_LT: RK_BC_BIN(x < y ? CT(1) : CT(0));
            case RK_BC_LE: RK_BC_BIN(x <= y ? CT(1) : CT(0));
            case RK_BC_GT: RK_BC_BIN(x > y ? CT(1) : CT(0));
            case RK_BC_GE: RK_BC_BIN(x >= y ? CT(1) : CT(0));
            case RK_BC_EQ: RK_BC_BIN(x == y ? CT(1) : CT(0));
            case RK_BC_NE: RK_BC_BIN(x != y ? CT(1) : CT(0));
            case RK_BC_AND: RK_BC_BIN(((x != CT(0)) && (y != CT(0))) ? CT(1) : CT(0));
            case RK_BC_OR: RK_BC_BIN(((x != CT(0)) || (y != CT(0))) ? CT(1) : CT(0));
            case RK_BC_NOT: RK_BC_UN(x == CT(0) ? CT(1) : CT(0));
            case RK_BC_IFELSE: {                // ifelse(c, a, b): c is the deepest of the three
#pragma unroll
                for (int j = 0; j < N; ++j) s0[j] = s2[j] != CT(0) ? s1[j] : s0[j];
                drop_second();
                drop_second();
            } break;
            default:                            // RK_BC_IDENTITY, or a token of one kind of program only
                if constexpr (std::is_floating_point<CT>::value) {
                    switch (tok) {
                        case RK_BC_DIV: RK_BC_BIN(x / y);
                        case RK_BC_SQRT: RK_BC_UN(sqrt(x));
                        case RK_BC_EXP: RK_BC_UN(exp(x));
                        case RK_BC_LOG: RK_BC_UN(log(x));
                        case RK_BC_INV: RK_BC_UN(CT(1) / x);
                        case RK_BC_ISNAN: RK_BC_UN(x != x ? CT(1) : CT(0));
                        case RK_BC_ROUND_F16: RK_BC_UN((CT)(half_t)x);
                        default:
                            if constexpr (FULL) {
                                switch (tok) {
                                    case RK_BC_POW: RK_BC_BIN(pow(x, y));
                                    case RK_BC_SIN: RK_BC_UN(sin(x));
                                    case RK_BC_COS: RK_BC_UN(cos(x));
                                    case RK_BC_TANH: RK_BC_UN(tanh(x));
                                    default: break;
                                }
                            }
                            break;
                    }
                } else {
                    switch (tok) {
                        case RK_BC_ISODD: RK_BC_UN(x & CT(1));
                        case RK_BC_ISEVEN: RK_BC_UN((x & CT(1)) ^ CT(1));
                        case RK_BC_ISNAN: RK_BC_UN(x * CT(0));
                        case RK_BC_WRAP_I32: RK_BC_UN((CT)(int32_t)x);
                        case RK_BC_WRAP_U32: RK_BC_UN((CT)(uint32_t)x);
                        case RK_BC_WRAP_I8: RK_BC_UN((CT)(int8_t)x);
                        case RK_BC_WRAP_U8: RK_BC_UN((CT)(uint8_t)x);
                        case RK_BC_WRAP_I16: RK_BC_UN((CT)(int16_t)x);
                        case RK_BC_WRAP_U16: RK_BC_UN((CT)(uint16_t)x);
                        default: break;
                    }
                }
                break;
        }
    }
#undef RK_BC_OPERAND
#undef RK_BC_UN
#undef RK_BC_BIN
#pragma unroll
    for (int j = 0; j < N; ++j) out[j] = s0[j];
}

}  // namespace rk
