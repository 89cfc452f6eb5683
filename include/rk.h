/*
 * rk.h -- C ABI of librk.so: hand-written gfx950 (MI355X) kernels for the array-kernel
 * layer behind AMDGPU.jl's ROCArray.
 *
 * Every entry point replaces one Julia method family of the reference (file:line given
 * at each declaration, relative to the AMDGPU.jl tree).  The Julia signatures stay as
 * they are; their bodies become a `ccall` of the functions below.
 *
 * Conventions (they mirror how the reference calls ROCm libraries,
 * src/hip/libhip.jl:5599-5610 and src/hip/error.jl:143-147):
 *   - plain pointers and sizes only; arrays are DENSE COLUMN-MAJOR device buffers
 *     described by (pointer, ndim, shape[ndim]); the pointer is what
 *     `Base.unsafe_convert(Ptr{T}, ::ROCArray)` yields (src/array.jl:353-354);
 *   - every call is asynchronous on the given hipStream_t (passed as void*), does not
 *     synchronise, does not allocate and does not retain caller pointers;
 *   - the return value is 0 (RK_SUCCESS), a hipError_t (1..9999) reported by the HIP
 *     runtime, or one of the RK_ERR_* codes (>= 10000); no exceptions, no errno, no abort;
 *   - zero-length inputs return RK_SUCCESS without launching (src/kernels/mapreduce.jl:91);
 *   - scalar arguments passed by pointer (`init`) are HOST pointers, read during the call.
 *
 * Workspace.  Reductions over many workgroups and the single-pass scan keep small
 * bookkeeping state (completion tickets, an epoch, per-tile descriptors, partials) in a
 * caller-owned device buffer.  Contract: allocate at least rk_workspace_bytes(...) bytes
 * (256-byte aligned), call rk_workspace_init() ONCE on it, and from then on pass it to
 * calls that are ordered on one stream at a time.  The kernels leave the bookkeeping
 * clean for the next call, so no per-call memset is needed.  One workspace per stream
 * corresponds to the reference's per-task library handles (src/cache.jl:102-137).
 */
#ifndef RK_H
#define RK_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define RK_API __attribute__((visibility("default")))
#else
#define RK_API
#endif

#define RK_VERSION 100          /* 0.1.0 */
#define RK_MAX_DIMS 8
#define RK_MAX_OPERANDS 8
#define RK_MAX_PROGRAM 48

/* ---- status codes -------------------------------------------------------------- */
enum {
    RK_SUCCESS = 0,
    /* 1..9999: hipError_t values passed through unchanged */
    RK_ERR_INVALID_ARGUMENT = 10001, /* null pointer, bad enum, ndim out of range, ...   */
    RK_ERR_UNSUPPORTED      = 10002, /* legal request outside the enumerated op set      */
    RK_ERR_WORKSPACE        = 10003, /* workspace missing, misaligned or too small       */
    RK_ERR_DIMENSION        = 10004, /* shapes do not agree (Julia: DimensionMismatch)   */
    RK_ERR_TOO_LARGE        = 10005, /* an extent exceeds what the kernels index         */
    RK_ERR_WAIT             = 10006  /* a kernel gave up a wait on another workgroup     */
};

/* ---- element types (Julia eltype <-> code) -------------------------------------- */
typedef enum {
    RK_F32 = 0,  /* Float32 */
    RK_F64 = 1,  /* Float64 */
    RK_I32 = 2,  /* Int32   */
    RK_I64 = 3,  /* Int64   */
    RK_U8  = 4,  /* Bool / UInt8 (one byte per element) */
    RK_U32 = 5,  /* UInt32  */
    RK_U64 = 6,  /* UInt64  */
    RK_F16 = 7,  /* Float16: rk_mapreduce (accumulating in Float32), rk_findminmax, rk_broadcast operands and
                  * destinations, rk_sort / rk_sortperm, rk_accumulate (scanned in Float32, rounded once at the store) */
    RK_I16 = 8,  /* Int16 */
    RK_I8  = 9,  /* Int8  */
    RK_U16 = 10  /* UInt16.  The three narrow integers: rk_mapreduce (sum / prod into Int64 or UInt64 as Base.add_sum
                  * widens them, max / min in their own type), rk_findminmax, rk_broadcast operands and destinations
                  * (integer programs compute in Int64 and store the low bits), rk_accumulate into their own type
                  * (scanned in 32 bits, the store keeps the low bits = the type's own wrap-around); Int16 also rk_sort /
                  * rk_sortperm.  Not rk_mapreduce_program (RK_ERR_UNSUPPORTED).  rk_reverse and rk_permutedims take an
                  * element SIZE, not a dtype, and so move any 1- or 2-byte element */
} rk_dtype;

/* f of mapreduce(f, op, A) */
typedef enum { RK_MAP_IDENTITY = 0, RK_MAP_ABS2 = 1, RK_MAP_ABS = 2 } rk_map;

/* op of mapreduce / accumulate.  Base.add_sum / mul_prod are ADD / MUL with a wider
 * output dtype chosen by the caller (Int32 -> Int64). */
/* RK_OP_AND / OR / XOR: the bitwise operators, in scans (rk_accumulate*) of integer element types and Bool only --
 * accumulate(&, A), accumulate(|, A), accumulate(xor, A); reductions return RK_ERR_UNSUPPORTED for them. */
typedef enum { RK_OP_ADD = 0, RK_OP_MUL = 1, RK_OP_MAX = 2, RK_OP_MIN = 3, RK_OP_AND = 4, RK_OP_OR = 5, RK_OP_XOR = 6 } rk_op;

/* which entry point a workspace is sized for */
typedef enum {
    RK_KIND_MAPREDUCE = 0, RK_KIND_FINDMINMAX = 1, RK_KIND_ACCUMULATE = 2, RK_KIND_FINDALL = 3
} rk_opkind;

/* ---- library ------------------------------------------------------------------- */
RK_API int32_t     rk_version(void);
RK_API const char* rk_status_string(int32_t status);

/* Bytes of workspace that a call of `kind` on an array of `ndim`/`shape` with element
 * type `dt` needs (dims_mask: bit d-1 set = Julia dim d is reduced; for accumulate the
 * single scanned dim).  For RK_KIND_ACCUMULATE `dt` is the OUTPUT dtype of the scan -- the
 * type the prefixes are carried in: cumsum of Bool into Int64 is sized with RK_I64, and
 * sizing it with the input dtype would give half the descriptor words.  For the *_strided
 * entry points pass the extents in the array's order of dims in memory.
 * Never fails: bad arguments return the generic minimum.
 * A buffer of RK_WORKSPACE_DEFAULT bytes serves every call up to 2^31 elements. */
#define RK_WORKSPACE_DEFAULT ((size_t)16 << 20)
RK_API size_t  rk_workspace_bytes(rk_opkind kind, rk_dtype dt, int ndim, const int64_t* shape,
                           uint32_t dims_mask);

/* Zero the bookkeeping area of a freshly allocated workspace (asynchronous on `stream`).
 * Call once per allocation, before its first use. */
RK_API int32_t rk_workspace_init(void* ws, size_t ws_bytes, void* stream);

/* Bounded waits.  The single-pass scan, the one-pass findall and the sort hand values from
 * workgroup to workgroup through the workspace (the sort: through its temporary); the
 * receiving side polls.  With a prepared workspace used by one call at a time such a wait
 * ends within microseconds.  A workspace that was never prepared, or that two calls use at
 * the same time, could make it wait for ever -- a hung GPU -- so every wait counts its
 * unsuccessful polls: after `rounds` of them (default 2^21, a second or two; environment
 * RK_WAIT_BUDGET) the kernel records the failure in the workspace, stops waiting and runs to
 * its end with meaningless results.  The record names the call that failed: the other
 * workgroups of that call give up with it, later calls on the same workspace are not touched
 * by it and run normally, and it stays readable until the workspace is prepared again.  A
 * binding reads it wherever it synchronises anyway (copy to the host, scalar fetch) and
 * raises.  No counterpart in the reference, whose kernels never wait on each other (it
 * launches one kernel per pass, src/kernels/mapreduce.jl:158-170).
 *   rk_set_wait_budget   sets the budget for later calls of this process (<= 0: the default)
 *                        and returns the previous one.
 *   rk_workspace_status  SYNCHRONISES `stream`, then returns RK_ERR_WAIT if any call on the
 *                        workspace gave up a wait since it was last prepared, else
 *                        RK_SUCCESS.  After RK_ERR_WAIT call rk_workspace_init again.
 *   rk_sort_status       the same for the temporary of rk_sort / rk_sortperm (no
 *                        preparation needed afterwards: every sort clears its temporary).
 *   rk_accumulate_static_status   the same for the library's own array behind
 *                        rk_accumulate_static on the current device; after RK_ERR_WAIT the
 *                        array has been prepared again before the call returns. */
RK_API int64_t rk_set_wait_budget(int64_t rounds);
RK_API int32_t rk_workspace_status(const void* ws, size_t ws_bytes, void* stream);
RK_API int32_t rk_sort_status(const void* tmp, size_t tmp_bytes, void* stream);
RK_API int32_t rk_accumulate_static_status(void* stream);

/* ---- mapreduce ------------------------------------------------------------------
 * Replaces GPUArrays.mapreducedim!(f, op, R, A; init)      src/kernels/mapreduce.jl:86-173
 * and its device kernels partial_mapreduce_device / reduce_group        :43-82, :8-34.
 *
 * A: `ndim`-dimensional column-major array of `in` elements.  Bit d-1 of `reduce_mask`
 * set = Julia dimension d is reduced; R has A's shape with every reduced dimension of
 * size 1 (mapreduce.jl:95-107) and element type `out`.  R is OVERWRITTEN with
 * op(init, reduction); `init` = host pointer to one `out` element, or NULL for op's
 * neutral element (0, 1, typemin, typemax).  One launch, no recursion, no allocation.
 * Supported (in -> out): same type for F32, F64, F16, I32, I64, U8, U32, U64 (Float16:
 * f in Float16, accumulation in Float32, one rounding at the end); I32/U8 -> I64 and
 * U32 -> U64 (add_sum widening).  MAX/MIN on floats follow Base.max/min (NaN propagates,
 * -0.0 < 0.0). */
RK_API int32_t rk_mapreduce(rk_map f, rk_op op, rk_dtype in, rk_dtype out,
                     const void* A, int ndim, const int64_t* shape, uint32_t reduce_mask,
                     void* R, const void* init,
                     void* ws, size_t ws_bytes, void* stream);

/* The same for wrapper arrays: `A` and / or `R` a transpose, PermutedDimsArray or reshape of a dense
 * array, as in the reference's own test  mapreducedim!(identity, +, transpose(R), A) === R
 *                                                        test/core/rocarray_base.jl:263-267
 * (the method takes any AnyROCArray destination, src/kernels/mapreduce.jl:86-89,172).
 * `A`, `R` point at the first element; `a_strides` / `r_strides` are element strides per dim (NULL =
 * dense column-major; entries of R's reduced dims are ignored).  A must be PERMUTED-DENSE: its strides
 * those of a dense array with the dims in some order (no gaps, no negative or zero strides); anything
 * else -- a view with gaps -- is RK_ERR_UNSUPPORTED (copy it first).  R may have any strides; when they
 * differ from where the kernels put the result, it is reduced into the workspace (at most 2.5 MiB of
 * results, else RK_ERR_UNSUPPORTED) and copied into R by the strided broadcast kernel. */
RK_API int32_t rk_mapreduce_strided(rk_map f, rk_op op, rk_dtype in, rk_dtype out,
                             const void* A, int ndim, const int64_t* shape, const int64_t* a_strides,
                             uint32_t reduce_mask, void* R, const int64_t* r_strides, const void* init,
                             void* ws, size_t ws_bytes, void* stream);

/* ---- mapreduce with f given as a program -----------------------------------------------
 * Replaces GPUArrays.mapreducedim!(f, op, R, A) for an f outside the rk_map list
 *                                                        src/kernels/mapreduce.jl:86-89
 * e.g. mapreduce(x -> x + 1, +, A; dims) (benchmarked in perf/array.jl:107-122), sum(f, A),
 * count(isodd, A), any(x -> x > 0, A).  f is a postfix program of rk_bc_token (declared with
 * the broadcast below) over the element -- operand token 0 -- and up to RK_MAP_MAX_CONSTS
 * constants -- operand tokens 1 ..; at most RK_MAP_MAX_TOKENS tokens and a value stack of
 * depth 4.  Float32 / Float64 elements compute in their own type, integer elements in Int64
 * (constants from const_i; the program holds RK_BC_WRAP_* where a 32-bit intermediate
 * matters), and the result is converted to `out`.
 * Supported (in -> out): F32 -> F32, F64 -> F64, I32 -> I32, I64 -> I64, I32 -> I64,
 * U8 -> I64; F32 -> I64 and F64 -> I64 with RK_OP_ADD only (counts).
 * Everything else as rk_mapreduce. */
#define RK_MAP_MAX_TOKENS 16
#define RK_MAP_MAX_CONSTS 4
#define RK_MAP_PROGRAM 3          /* the f of these calls, next to the rk_map values */
typedef struct {
    int32_t n_tokens;
    int32_t tokens[RK_MAP_MAX_TOKENS];
    int32_t n_consts;
    double  const_f[RK_MAP_MAX_CONSTS];   /* used when the elements are F32 / F64 */
    int64_t const_i[RK_MAP_MAX_CONSTS];   /* used when they are integers          */
} rk_map_program;
RK_API int32_t rk_mapreduce_program(const rk_map_program* f, rk_op op, rk_dtype in, rk_dtype out,
                      const void* A, int ndim, const int64_t* shape, uint32_t reduce_mask,
                      void* R, const void* init,
                      void* ws, size_t ws_bytes, void* stream);

/* ---- findmax / findmin -----------------------------------------------------------
 * Replaces the (value, CartesianIndex) tuple reduction that GPUArrays' findminmax sends
 * through mapreducedim!                                    src/kernels/mapreduce.jl:86
 * (benchmarked in perf/array.jl:50-53).
 *
 * vals: A's shape with reduced dims of size 1, element type `in`.
 * cart_idx: for each output element `ndim` consecutive Int64 = the 1-based CartesianIndex
 * of the winner in A (memory layout of Array{CartesianIndex{ndim}}).  Ties -> smallest
 * column-major index; the first NaN wins; +0.0 > -0.0 (Base.isless order).
 * Either output pointer may be NULL to skip it. */
RK_API int32_t rk_findminmax(int32_t want_max, rk_dtype in,
                      const void* A, int ndim, const int64_t* shape, uint32_t reduce_mask,
                      void* vals, int64_t* cart_idx,
                      void* ws, size_t ws_bytes, void* stream);

/* The same for wrapper arrays -- findmax(transpose(A); dims), findmin(PermutedDimsArray(A, p); dims) -- which the
 * reference sends through the same generic findminmax of GPUArrays (src/kernels/mapreduce.jl:86-173 underneath).
 * `shape` and `a_strides` (in elements) describe the wrapper; it must be a permutation of a dense array's dims.  The
 * index goes out in the wrapper's coordinates, the outputs are dense in the wrapper's shape.  Served when the kept dims
 * and the reduced dims each keep their relative order in memory (a transposed matrix along either dim, any wrapper with
 * one reduced dim whose kept dims are in order): then "first of equal winners" and the output layout agree with the
 * wrapper's column-major order.  Anything else is RK_ERR_UNSUPPORTED (copy the wrapper first). */
RK_API int32_t rk_findminmax_strided(int32_t want_max, rk_dtype in,
                      const void* A, int ndim, const int64_t* shape, const int64_t* a_strides, uint32_t reduce_mask,
                      void* vals, int64_t* cart_idx,
                      void* ws, size_t ws_bytes, void* stream);

/* ---- accumulate / cumsum / cumprod -------------------------------------------------
 * Replaces Base.accumulate!/accumulate/cumsum/cumprod(::AnyROCArray)
 *                                                        src/kernels/accumulate.jl:1-8
 * (forwarders into AcceleratedKernels.accumulate!).
 *
 * Scans along Julia dimension `dim` (1-based; dim > ndim copies, with init folded in).
 * `out` may alias `in` when the dtypes agree.  inclusive != 0: out[k] = init op a[1] op ..
 * op a[k]; inclusive == 0: out[k] = init op a[1] op .. op a[k-1].  `init` = host pointer to
 * one `out` element or NULL for the neutral element.  Integer arithmetic wraps.
 * Supported (in -> out): same type (every rk_dtype); U8 -> I64, U8 -> I32 (Bool counts). ADD and MUL;
 * MAX / MIN, and AND / OR / XOR on integer types, for same-type scans. */
RK_API int32_t rk_accumulate(rk_op op, rk_dtype in, rk_dtype out,
                      const void* in_ptr, void* out_ptr,
                      int ndim, const int64_t* shape, int dim, int32_t inclusive,
                      const void* init,
                      void* ws, size_t ws_bytes, void* stream);

/* The same for wrapper arrays (cumsum!(transpose(B), transpose(A)), accumulate! on a
 * PermutedDimsArray): input and output permuted-dense (see rk_mapreduce_strided) with the SAME order of
 * dims in memory; anything else is RK_ERR_UNSUPPORTED.  `dim` is the logical dimension. */
RK_API int32_t rk_accumulate_strided(rk_op op, rk_dtype in, rk_dtype out,
                              const void* in_ptr, void* out_ptr,
                              int ndim, const int64_t* shape, const int64_t* in_strides,
                              const int64_t* out_strides, int dim, int32_t inclusive,
                              const void* init, void* ws, size_t ws_bytes, void* stream);

/* ---- accumulate without a caller workspace ------------------------------------------------
 * No counterpart in the reference.  For callers that cannot allocate device memory at all --
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc -- and so
 * cannot bring the workspace rk_accumulate asks for: the same scan, with its bookkeeping
 * (tile counter, look-back descriptors, slice totals) in a device array of
 * RK_STATIC_SCRATCH_BYTES that is part of the library image, one copy per GPU, held until the
 * process ends.  Arguments and results as rk_accumulate.  Calls whose bookkeeping would not fit
 * (rk_workspace_bytes(RK_KIND_ACCUMULATE, ...) > RK_STATIC_SCRATCH_BYTES) return
 * RK_ERR_TOO_LARGE.  Calls no hipMalloc / hipFree.  Every call on a GPU uses that GPU's one
 * array: calls that overlap in time on one GPU (two streams, two threads) race and must be
 * ordered by the caller.  The first call on each device prepares the array with a small kernel
 * on `stream` and waits for it (so that calls on other streams find it prepared); it must not be
 * made while that stream is being captured (RK_ERR_WORKSPACE).  A give-up of a bounded wait
 * is read with rk_accumulate_static_status. */
#define RK_STATIC_SCRATCH_BYTES ((size_t)16 << 20)
RK_API int32_t rk_accumulate_static(rk_op op, rk_dtype in, rk_dtype out,
                             const void* in_ptr, void* out_ptr,
                             int ndim, const int64_t* shape, int dim, int32_t inclusive,
                             const void* init, void* stream);

/* ---- fused broadcast ---------------------------------------------------------------
 * Replaces copyto!(dest, ::Broadcasted{<:ROCArrayStyle})              src/broadcast.jl:3-35
 * i.e. GPUArrays' broadcast kernel launched through the KernelAbstractions functor
 *                                                              src/ROCKernels.jl:107-129.
 *
 * The Broadcasted tree is flattened to a postfix program over up to RK_MAX_OPERANDS
 * operands.  An array operand has `ndim` <= dest's ndim and each extent either equal to
 * dest's or 1 (extruded: stride 0, what Broadcast.preprocess/Extruded does); missing
 * trailing dims count as 1.  A scalar operand is passed by value. */
typedef enum {
    /* tokens 0 .. RK_MAX_OPERANDS-1 push that operand */
    RK_BC_ADD = 32, RK_BC_SUB, RK_BC_MUL, RK_BC_DIV, RK_BC_MAX, RK_BC_MIN, RK_BC_POW,
    RK_BC_FMA,                 /* muladd(a, b, c): pops c, b, a                         */
    RK_BC_NEG = 64, RK_BC_ABS, RK_BC_ABS2, RK_BC_SQRT, RK_BC_EXP, RK_BC_LOG, RK_BC_SIN,
    RK_BC_COS, RK_BC_TANH, RK_BC_INV, RK_BC_IDENTITY,
    /* predicates and logic: the result is 1 or 0 in the compute type (a Bool once stored to a U8 dest);
     * AND / OR / NOT / IFELSE read "nonzero" as true */
    RK_BC_LT = 96, RK_BC_LE, RK_BC_GT, RK_BC_GE, RK_BC_EQ, RK_BC_NE, RK_BC_AND, RK_BC_OR,
    RK_BC_IFELSE = 112,        /* ifelse(c, a, b): pops b, a, c                          */
    RK_BC_NOT = 128, RK_BC_ISODD, RK_BC_ISEVEN,     /* ISODD / ISEVEN: integer programs     */
    RK_BC_ISNAN,
    RK_BC_WRAP_I32,            /* integer programs: sign-extend the low 32 bits, i.e. the Int32 value Julia
                                * holds at this point (needed before order-sensitive tokens only)      */
    RK_BC_WRAP_U32,            /* the same, zero-extending (UInt32)                                    */
    RK_BC_ROUND_F16,           /* Float32 programs over Float16 arrays: round to Float16 and back, after every
                                * operation whose Julia result is a Float16 (Julia computes Float16 arithmetic in
                                * Float32 and rounds each result)                                       */
    RK_BC_WRAP_I8, RK_BC_WRAP_U8, RK_BC_WRAP_I16, RK_BC_WRAP_U16     /* as WRAP_I32 / WRAP_U32, for the narrow integers */
} rk_bc_token;

typedef struct {
    const void* ptr;              /* device pointer; NULL for a scalar operand           */
    int32_t     dtype;            /* rk_dtype of the array elements / of the scalar      */
    int32_t     ndim;             /* 0 for scalars                                       */
    int64_t     shape[RK_MAX_DIMS];
    double      scalar_f;         /* scalar value when dtype is F32/F64                  */
    int64_t     scalar_i;         /* scalar value when dtype is an integer type          */
    int32_t     strided;          /* != 0: `strides` below describe the array (a view, a
                                   * transpose, a PermutedDimsArray); 0: dense column-major */
    int32_t     reserved;
    int64_t     strides[RK_MAX_DIMS]; /* element strides per dim; may be negative          */
} rk_operand;

typedef struct {
    int32_t    compute;           /* rk_dtype every operand is converted to: F32, F64, or
                                   * I64 for integer programs (no / ^ or math functions; the
                                   * store keeps the low bits, i.e. Int32 results wrap as in
                                   * Julia)                                                */
    int32_t    n_operands;
    rk_operand operands[RK_MAX_OPERANDS];
    int32_t    n_tokens;
    int32_t    tokens[RK_MAX_PROGRAM];
} rk_program;

RK_API int32_t rk_broadcast(const rk_program* prog, void* dest, rk_dtype dest_dtype,
                     int ndim, const int64_t* shape, void* stream);
/* The same with a destination that is a strided view (`@view(C[2:5, :]) .= ...`,
 * `transpose(C) .= ...`): `dest` points at its first element, `dest_strides` are its element
 * strides per dim (NULL = dense).  Distinct index tuples must address distinct elements. */
RK_API int32_t rk_broadcast_strided(const rk_program* prog, void* dest, rk_dtype dest_dtype,
                             int ndim, const int64_t* shape, const int64_t* dest_strides,
                             void* stream);

/* ---- volumerhs -----------------------------------------------------------------------
 * Replaces `@roc groupsize=(5,5) gridsize=nelem volumerhs!(rhs, Q, vgeo, gravity, D, nelem)`
 *                                                   perf/volumerhs.jl:42-176, :200-201.
 * N = 4 (Nq = 5), 5 states, 14 metric fields, Float32, like the reference's benchmark:
 * rhs, Q: (5,5,5,5,nelem); vgeo: (5,5,5,14,nelem); D: (5,5); all column-major.
 * rhs is accumulated into (+=).  rhs must not alias Q or vgeo. */
RK_API int32_t rk_volumerhs_f32(float* rhs, const float* Q, const float* vgeo, float gravity,
                         const float* D, int64_t nelem, void* stream);

/* ---- findall scatter (caller of the scan) -----------------------------------------------
 * Replaces the scatter kernel `_ker!` of Base.findall(::AnyROCArray{Bool})
 *                                                        src/kernels/indexing.jl:16-31.
 * `indices` = inclusive Int64 cumsum of the flattened `bools` (rk_accumulate U8 -> I64).
 * Writes, for every true element, its 1-based CartesianIndex (`ndim` Int64, or the linear
 * index when ndim == 1) to ys[indices[i]-1]. */
RK_API int32_t rk_findall_scatter(const uint8_t* bools, const int64_t* indices, int64_t* ys,
                           int ndim, const int64_t* shape, void* stream);

/* ---- findall in one pass ------------------------------------------------------------------
 * Replaces the whole body of Base.findall(::AnyROCArray{Bool})  src/kernels/indexing.jl:8-36
 * after the count is known: the Int64 cumsum (`:10`), the scatter kernel (`:16-31`) and the
 * temporary they share (`:33`) become one pass that reads each Bool once and writes the indices.
 * `ys` must hold count(bools) entries (the caller gets the count from
 * rk_mapreduce(RK_MAP_IDENTITY, RK_OP_ADD, RK_U8 -> RK_I64), the `indices[end]` of `:12`):
 * `ndim` Int64 per entry (1-based CartesianIndex, column-major), or the linear index when
 * ndim <= 1; entries are in column-major order of the elements.  Only bit 0 of a Bool byte is
 * looked at.  If `count_out` is not NULL it receives the number of entries written (device
 * pointer, Int64).  Needs the workspace (RK_KIND_FINDALL). */
RK_API int32_t rk_findall(const uint8_t* bools, int ndim, const int64_t* shape, int64_t* ys,
                   int64_t* count_out, void* ws, size_t ws_bytes, void* stream);

/* ---- gather along the last dimension ---------------------------------------------------------
 * y[i, j] = x[i, idx[j]] for i in 1:inner, j in 1:nidx (idx 1-based, Int64; x has `nsrc` slices
 * of `inner` elements).  Serves logical indexing `x[mask]`, `x[:, mask]`, `x[:, :, mask]`
 * (test/hip_rocarray/indexing.jl:5-18) once  Base.to_index(::ROCArray, ::AbstractArray{Bool})
 * src/kernels/indexing.jl:1  has produced idx = findall(mask); the reference leaves the gather to
 * GPUArrays' generic indexing kernel.  Elements are opaque (`elsize` = 1, 2, 4, 8 or 16). */
RK_API int32_t rk_gather_slices(const void* x, const int64_t* idx, void* y, size_t elsize,
                         int64_t inner, int64_t nidx, int64_t nsrc, void* stream);

/* ---- reverse / reverse! -------------------------------------------------------------------
 * Replaces both `_reverse!` kernels of src/kernels/reverse.jl: out of place (`:59-88`, y != x)
 * and in place (`:92-122`, y == x; partially overlapping x and y are not allowed).
 * Elements are opaque: `elsize` bytes each (1, 2, 4, 8 or 16).  Bit d-1 of `rev_mask` set =
 * Julia dim d is flipped (`dims=:` = all bits; extents of 1 never flip, `:67`).  rev_mask == 0
 * with y != x is a plain copy, which serves the head and tail copies of
 * `reverse(x, start, stop)` (`:11-12`); the partial reverse itself is a call on the view's
 * pointer.  No workspace. */
RK_API int32_t rk_reverse(const void* x, void* y, size_t elsize, int ndim, const int64_t* shape,
                   uint32_t rev_mask, void* stream);

/* ---- permutedims / permutedims! -------------------------------------------------------------
 * dst = permutedims(src, perm): dst[i_perm[1], ..., i_perm[N]] = src[i_1, ..., i_N], i.e.
 * size(dst, k) == shape[perm[k]-1]; `perm` is 1-based like Julia's.  The reference has no
 * kernel of its own for this: it runs GPUArrays' generic one-element-per-work-item kernel
 * (benchmarked in perf/array.jl:151-155).  Elements are opaque (`elsize` = 1, 2, 4, 8 or 16
 * bytes); src and dst are dense, column-major and must not overlap.  No workspace. */
RK_API int32_t rk_permutedims(const void* src, void* dst, size_t elsize, int ndim,
                       const int64_t* shape, const int32_t* perm, void* stream);

/* ---- sort! / sortperm! of vectors ------------------------------------------------------------
 * Replace AK.sort! / AK.sortperm! behind  src/kernels/sorting.jl:1-3  for the default order
 * (`lt = isless`, `by = identity`) and `rev`; custom `lt` / `by` closures cannot cross a C ABI
 * (the caller keeps its own path for them).  Element types: Float16/32/64, Int16/32/64 (the types
 * of test/hip_rocarray/sorting.jl).  Order = Base.isless: -0.0 before 0.0, NaN last.  The sorted
 * array is a permutation of the input bit for bit: NaNs keep sign and payload (their order among
 * themselves is by bit pattern).  Stable: sortperm keeps equal keys -- all NaNs count as equal --
 * in index order, also with rev != 0, like Base.
 *   rk_sort      sorts `keys` in place.
 *   rk_sortperm  leaves `keys` untouched and writes the 1-based permutation (Int64) to
 *                `perm_out`; unlike `sortperm!(ix, x)` it does not read an initial `ix`
 *                (the reference always passes 1:n, src/kernels/sorting.jl:3).
 * `tmp`: caller-owned, 256-byte aligned, at least rk_sort_tmp_bytes(dt, n, with_perm) bytes, any
 * contents; it is the ping-pong buffer plus bookkeeping, cleared by the call itself.  n < 2^31. */
RK_API size_t  rk_sort_tmp_bytes(rk_dtype dt, int64_t n, int32_t with_perm);
RK_API int32_t rk_sort(rk_dtype dt, void* keys, int64_t n, int32_t rev, void* tmp, size_t tmp_bytes,
                void* stream);
RK_API int32_t rk_sortperm(rk_dtype dt, const void* keys, int64_t* perm_out, int64_t n, int32_t rev,
                    void* tmp, size_t tmp_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RK_H */
