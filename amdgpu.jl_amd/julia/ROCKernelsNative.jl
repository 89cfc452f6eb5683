# ROCKernelsNative.jl -- the reference-side binding of librk.so.
#
# Load AFTER AMDGPU.jl:  `using AMDGPU; include("ROCKernelsNative.jl"); ROCKernelsNative.enable!()`
# The Julia API surface does not change.  The method families below get a more specific method whose body
# is a `ccall` into the hand-written gfx950 kernels (C ABI: include/rk.h); whatever the native layer does not
# enumerate (arbitrary closures, wrapper types, exotic eltypes) falls through to the stock GPUArrays /
# AcceleratedKernels methods by `invoke`.
#
#   replaced method family                                   reference location
#   GPUArrays.mapreducedim!(f, op, R::AnyROCArray, A; init)  src/kernels/mapreduce.jl:86-173
#   Base.accumulate!/accumulate/cumsum/cumprod               src/kernels/accumulate.jl:1-8
#   Base.copyto!(dest, ::Broadcasted{<:ROCArrayStyle})       src/broadcast.jl:3-35 (+ GPUArrays _copyto!)
#   findmax/findmin(A; dims), A a ROCArray or a transpose / PermutedDimsArray of one   GPUArrays findminmax -> mapreducedim!
#   volumerhs!(rhs, Q, vgeo, gravity, D, nelem)              perf/volumerhs.jl:200-201
#
# This file is shipped as text: no Julia runtime exists where this repository is built and tested, so it is
# exercised only where `julia` and AMDGPU.jl are installed.  The Python host mirror in this package makes
# exactly the same calls and is what the test-suite drives.
module ROCKernelsNative

using AMDGPU
using AMDGPU: ROCArray, AnyROCArray, ROCArrayStyle, HIP
import GPUArrays
import LinearAlgebra
import Base.Broadcast: Broadcasted

const librk = Ref{String}(joinpath(@__DIR__, "..", "librk.so"))

# ---- status handling: integer status -> exception, like AMDGPU's @check (src/utils.jl:226-242) -------------
struct RKError <: Exception
    code::Int32
end
function Base.showerror(io::IO, e::RKError)
    msg = unsafe_string(ccall((:rk_status_string, librk[]), Cstring, (Int32,), e.code))
    print(io, "RKError($(e.code)): $msg")
end
const RK_ERR_UNSUPPORTED = Int32(10002)
const RK_ERR_WORKSPACE = Int32(10003)
const RK_ERR_DIMENSION = Int32(10004)
const RK_ERR_TOO_LARGE = Int32(10005)
const RK_ERR_WAIT = Int32(10006)
# A legal request the library does not take -- an operation outside its set, an extent beyond what its kernels
# index, a workspace it cannot size -- is declined, not an error: the caller runs the stock method instead.
declined(status::Int32) = status == RK_ERR_UNSUPPORTED || status == RK_ERR_TOO_LARGE || status == RK_ERR_WORKSPACE
@inline function check(status::Int32)
    status == 0 && return nothing
    status == RK_ERR_DIMENSION && throw(DimensionMismatch("librk: array extents do not agree"))
    throw(RKError(status))
end

# ---- enums of include/rk.h ----------------------------------------------------------------------------------
rk_dtype(::Type{Float32}) = Cint(0); rk_dtype(::Type{Float64}) = Cint(1)
rk_dtype(::Type{Int32}) = Cint(2);   rk_dtype(::Type{Int64}) = Cint(3)
rk_dtype(::Type{Bool}) = Cint(4);    rk_dtype(::Type{UInt8}) = Cint(4)
rk_dtype(::Type{UInt32}) = Cint(5);  rk_dtype(::Type{UInt64}) = Cint(6)
rk_dtype(::Type{Float16}) = Cint(7); rk_dtype(::Type{Int16}) = Cint(8)
rk_dtype(::Type{Int8}) = Cint(9);    rk_dtype(::Type{UInt16}) = Cint(10)
rk_dtype(::Type) = nothing
rk_map(::typeof(identity)) = Cint(0); rk_map(::typeof(abs2)) = Cint(1); rk_map(::typeof(abs)) = Cint(2)
rk_map(_) = nothing
rk_op(::typeof(+)) = Cint(0); rk_op(::typeof(Base.add_sum)) = Cint(0)
rk_op(::typeof(*)) = Cint(1); rk_op(::typeof(Base.mul_prod)) = Cint(1)
rk_op(::typeof(max)) = Cint(2); rk_op(::typeof(min)) = Cint(3)
rk_op(::typeof(&)) = Cint(4); rk_op(::typeof(|)) = Cint(5); rk_op(::typeof(xor)) = Cint(6)    # scans of integers and Bools only:
rk_op(_) = nothing                                                                           # reductions decline them

# ---- one workspace per (device, stream): the analogue of the per-task library handles (src/cache.jl) --------
const WORKSPACE_BYTES = 16 << 20
const workspaces = Dict{Tuple{Int,Ptr{Cvoid}},ROCArray{UInt8,1}}()
const workspaces_lock = ReentrantLock()
stream_ptr() = Base.unsafe_convert(Ptr{Cvoid}, AMDGPU.stream().stream)     # hipStream_t of the task-local stream
function workspace(minbytes::Integer = 0)
    key = (AMDGPU.device_id(AMDGPU.device()), stream_ptr())
    lock(workspaces_lock) do
        ws = get(workspaces, key, nothing)
        if ws === nothing || length(ws) < minbytes
            ws = ROCArray{UInt8}(undef, max(WORKSPACE_BYTES, 2minbytes))
            check(ccall((:rk_workspace_init, librk[]), Int32, (Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                        pointer(ws), length(ws), stream_ptr()))
            workspaces[key] = ws
        end
        ws
    end
end

# ---- give-ups of bounded waits ---------------------------------------------------------------------------------
# The scans across rows, the scan of 8-byte / unaligned lines and sorts of up to 2^20 keys wait on other workgroups with
# a budget; a kernel that runs out of it records that in the workspace (the sort: in its temporary) and finishes with
# meaningless results.  The records are read where the host waits for the device anyway -- Array(x), a scalar fetch --
# for every workspace and sort temporary such a kernel has used on the task's stream since the last look; a give-up
# prepares the workspace again and throws.  (The single-pass scan of long lines and findall never give up.)
const waiting = Set{Tuple{Int,Ptr{Cvoid}}}()                                  # streams whose workspace a waiting kernel has used
const sort_tmps = Dict{Tuple{Int,Ptr{Cvoid}},Vector{ROCArray{UInt8,1}}}()     # temporaries of small sorts, record unread
note_waiting_call() = lock(() -> push!(waiting, (AMDGPU.device_id(AMDGPU.device()), stream_ptr())), workspaces_lock)
function note_sort(tmp::ROCArray{UInt8,1}, n::Integer)
    n > (1 << 20) && return AMDGPU.unsafe_free!(tmp)       # large sorts count before every pass and wait for nobody
    key = (AMDGPU.device_id(AMDGPU.device()), stream_ptr())
    pending = lock(() -> push!(get!(sort_tmps, key, ROCArray{UInt8,1}[]), tmp), workspaces_lock)
    length(pending) > 16 && check_waits()                  # a long run of sorts without a fetch: read rather than hoard
    return nothing
end
function check_waits()
    key = (AMDGPU.device_id(AMDGPU.device()), stream_ptr())
    failed = false
    ws, tmps = lock(workspaces_lock) do
        w = key in waiting ? get(workspaces, key, nothing) : nothing
        delete!(waiting, key)
        (w, pop!(sort_tmps, key, ROCArray{UInt8,1}[]))
    end
    if ws !== nothing
        st = ccall((:rk_workspace_status, librk[]), Int32, (Ptr{Cvoid}, Csize_t, Ptr{Cvoid}), pointer(ws), length(ws), stream_ptr())
        if st == RK_ERR_WAIT
            check(ccall((:rk_workspace_init, librk[]), Int32, (Ptr{Cvoid}, Csize_t, Ptr{Cvoid}), pointer(ws), length(ws), stream_ptr()))
            failed = true
        else
            check(st)
        end
    end
    for tmp in tmps
        st = ccall((:rk_sort_status, librk[]), Int32, (Ptr{Cvoid}, Csize_t, Ptr{Cvoid}), pointer(tmp), sizeof(tmp), stream_ptr())
        AMDGPU.unsafe_free!(tmp)
        st == RK_ERR_WAIT ? (failed = true) : check(st)
    end
    failed && throw(RKError(RK_ERR_WAIT))
    return nothing
end
# Array(x) and every scalar fetch copy device memory to the host, i.e. synchronise: the place to look.
function enable_wait_checks!()
    @eval function Base.Array(x::ROCArray{T,N}) where {T,N}
        check_waits()
        return copyto!(Array{T,N}(undef, size(x)), x)
    end
end

dense(A::ROCArray) = true          # dense column-major storage: (pointer, dims) describes it completely
dense(_) = false
# wrappers over a ROCArray that are (pointer, size, strides) triples: operands / destinations of the *_strided entry points
const ROCWrapper{T,N} = Union{SubArray{T,N,<:ROCArray}, LinearAlgebra.Transpose{T,<:ROCArray{T}},
                              PermutedDimsArray{T,N,<:Any,<:Any,<:ROCArray}}
is_strided_wrapper(x) = x isa ROCWrapper && eltype(x) <: Real && applicable(strides, x)
const ROCStrided{T,N} = Union{ROCArray{T,N},ROCWrapper{T,N}}
strides64(A, N) = Int64[k <= ndims(A) ? stride(A, k) : 0 for k in 1:N]

# ---- mapreducedim! ------------------------------------------------------------------------------------------
function native_mapreducedim!(f, op, R::ROCArray{TR}, A::ROCArray{TA,N}, init) where {TR,TA,N}
    Base.check_reducedims(R, A)
    isempty(A) && return true
    mask = UInt32(0)
    for d in 1:N
        size(R, d) == size(A, d) || (mask |= UInt32(1) << (d - 1))
    end
    ws = workspace()
    shape = Int64[size(A)...]
    initref = init === nothing ? C_NULL : Ref(convert(TR, init))
    GC.@preserve R A ws shape initref begin
        st = ccall((:rk_mapreduce, librk[]), Int32,
                   (Cint, Cint, Cint, Cint, Ptr{Cvoid}, Cint, Ptr{Int64}, UInt32, Ptr{Cvoid}, Ptr{Cvoid},
                    Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                   rk_map(f), rk_op(op), rk_dtype(TA), rk_dtype(TR), pointer(A), N, shape, mask, pointer(R),
                   initref === C_NULL ? C_NULL : Base.unsafe_convert(Ptr{Cvoid}, initref),
                   pointer(ws), length(ws), stream_ptr())
    end
    declined(st) && return false
    check(st)
    return true
end

# R or A a transpose / PermutedDimsArray / contiguous view, e.g. mapreducedim!(identity, +, transpose(R), A): the
# library renumbers the dims of permuted-dense arrays and declines (-> stock method) views with gaps
function native_mapreducedim_strided!(f, op, R::ROCStrided{TR}, A::ROCStrided{TA}, init) where {TR,TA}
    N = ndims(A)                 # (not a static parameter: a Transpose does not bind the alias's N)
    Base.check_reducedims(R, A)
    isempty(A) && return true
    mask = UInt32(0)
    for d in 1:N
        size(R, d) == size(A, d) || (mask |= UInt32(1) << (d - 1))
    end
    ws = workspace()
    shape = Int64[size(A)...]
    as, rs = strides64(A, N), strides64(R, N)
    initref = init === nothing ? C_NULL : Ref(convert(TR, init))
    GC.@preserve R A ws shape as rs initref begin
        st = ccall((:rk_mapreduce_strided, librk[]), Int32,
                   (Cint, Cint, Cint, Cint, Ptr{Cvoid}, Cint, Ptr{Int64}, Ptr{Int64}, UInt32, Ptr{Cvoid}, Ptr{Int64},
                    Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                   rk_map(f), rk_op(op), rk_dtype(TA), rk_dtype(TR), pointer(A), N, shape, as, mask, pointer(R), rs,
                   initref === C_NULL ? C_NULL : Base.unsafe_convert(Ptr{Cvoid}, initref),
                   pointer(ws), length(ws), stream_ptr())
    end
    declined(st) && return false
    check(st)
    return true
end

# ---- closures for f: traced on a symbolic element into an rk_map_program -----------------------------------------------
# f(MapSym) runs ordinary Julia code; every operator on a MapSym appends rk_bc_token values instead of computing.
# Token 0 is the element, tokens 1.. the scalars f closes over.  What the tracer cannot follow -- `if` on a value,
# functions without a method for MapSym -- throws, and the stock mapreducedim! runs instead.
struct RKMapProgram
    n_tokens::Int32; tokens::NTuple{16,Int32}; n_consts::Int32; const_f::NTuple{4,Float64}; const_i::NTuple{4,Int64}
end
struct MapSym{T} <: Real                # T: the Julia type the value would have
    toks::Vector{Int32}
    consts::Vector{Any}                 # shared by every node of one trace
end
operand!(s::MapSym, c::Union{Float32,Float64,Int32,Int64,UInt32,Bool}) = begin
    k = findfirst(==(c), s.consts)
    k === nothing && (push!(s.consts, c); k = length(s.consts))
    k > 4 && throw(Unsupported())
    Int32[k]
end
# Integer programs compute in Int64.  Where Julia's value is an Int32 / UInt32 -- the result of arithmetic on such
# values -- a wrap token (RK_BC_WRAP_I32 = 132, RK_BC_WRAP_U32 = 133) restores it, so comparisons, max / min and the
# widening sum see what Julia's wrapping arithmetic produces (mapreduce(x -> x + 1, +, ::ROCArray{Int32})).
wrap_tokens(::Type{Int32}) = Int32[132]
wrap_tokens(::Type{UInt32}) = Int32[133]
wrap_tokens(::Type) = Int32[]
for (f, tok) in ((:+, 32), (:-, 33), (:*, 34), (:/, 35), (:max, 36), (:min, 37), (:<, 96), (:<=, 97), (:>, 98), (:>=, 99),
                 (:(==), 100), (:!=, 101), (:&, 102), (:|, 103))
    R = tok >= 96 ? :(Bool) : tok == 35 ? :(typeof(one(A) / one(B))) : :(Base.promote_op($f, A, B))
    W = tok <= 34 ? :(wrap_tokens($R)) : :(Int32[])           # + - * can leave the 32-bit range
    @eval Base.$f(a::MapSym{A}, b::MapSym{B}) where {A,B} = MapSym{$R}(vcat(a.toks, b.toks, Int32($tok), $W), a.consts)
    @eval Base.$f(a::MapSym{A}, b::B) where {A,B<:Union{Float32,Float64,Int32,Int64,UInt32,Bool}} =
        MapSym{$R}(vcat(a.toks, operand!(a, b), Int32($tok), $W), a.consts)
    @eval Base.$f(a::A, b::MapSym{B}) where {A<:Union{Float32,Float64,Int32,Int64,UInt32,Bool},B} =
        MapSym{$R}(vcat(operand!(b, a), b.toks, Int32($tok), $W), b.consts)
end
for (f, tok) in ((:-, 64), (:abs, 65), (:abs2, 66), (:sqrt, 67), (:exp, 68), (:log, 69), (:inv, 73), (:!, 128), (:isodd, 129),
                 (:iseven, 130), (:isnan, 131))
    R = tok >= 128 ? :(Bool) : :(Base.promote_op($f, A))
    W = tok in (64, 65, 66) ? :(wrap_tokens($R)) : :(Int32[])  # -x, abs(x), abs2(x) of typemin(Int32) wrap
    @eval Base.$f(a::MapSym{A}) where {A} = MapSym{$R}(vcat(a.toks, Int32($tok), $W), a.consts)
end
Base.ifelse(c::MapSym{Bool}, a::MapSym{A}, b::MapSym{B}) where {A,B} =
    MapSym{promote_type(A, B)}(vcat(c.toks, a.toks, b.toks, Int32(112)), c.consts)

function trace_map(f, ::Type{T}) where {T}
    consts = Any[]
    y = f(MapSym{T}(Int32[0], consts))
    y isa MapSym || throw(Unsupported())
    R = typeof(y).parameters[1]
    toks = y.toks
    # (integer programs run in Int64; Int32 / UInt32 intermediates carry their wrap tokens, see wrap_tokens)
    T <: AbstractFloat && !all(c -> c isa T || c isa Integer, consts) && throw(Unsupported())      # 0.5 over Float32: a Float64 map
    length(toks) <= 16 || throw(Unsupported())
    cf = ntuple(k -> k <= length(consts) ? Float64(consts[k]) : 0.0, 4)
    ci = ntuple(k -> k <= length(consts) && !(consts[k] isa AbstractFloat) ? Int64(consts[k]) : Int64(0), 4)
    return Ref(RKMapProgram(length(toks), ntuple(i -> i <= length(toks) ? toks[i] : Int32(0), 16), length(consts), cf, ci)), R
end

function native_mapreducedim_closure!(f, op, R::ROCArray{TR}, A::ROCArray{TA,N}, init) where {TR,TA,N}
    prog, TM = try trace_map(f, TA) catch; return false end
    TR === Base.promote_op(op, TM, TM) || return false
    Base.check_reducedims(R, A)
    isempty(A) && return true
    mask = UInt32(0)
    for d in 1:N
        size(R, d) == size(A, d) || (mask |= UInt32(1) << (d - 1))
    end
    ws = workspace()
    shape = Int64[size(A)...]
    initref = init === nothing ? C_NULL : Ref(convert(TR, init))
    GC.@preserve R A ws shape initref prog begin
        st = ccall((:rk_mapreduce_program, librk[]), Int32,
                   (Ref{RKMapProgram}, Cint, Cint, Cint, Ptr{Cvoid}, Cint, Ptr{Int64}, UInt32, Ptr{Cvoid}, Ptr{Cvoid},
                    Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                   prog, rk_op(op), rk_dtype(TA), rk_dtype(TR), pointer(A), N, shape, mask, pointer(R),
                   initref === C_NULL ? C_NULL : Base.unsafe_convert(Ptr{Cvoid}, initref),
                   pointer(ws), length(ws), stream_ptr())
    end
    declined(st) && return false
    check(st)
    return true
end

function enable_mapreduce!()
    @eval function GPUArrays.mapreducedim!(f::F, op::OP, R::ROCArray{TR}, A::ROCArray{TA}; init=nothing) where {F,OP,TR,TA}
        if rk_map(f) !== nothing && rk_op(op) !== nothing && rk_dtype(TR) !== nothing && rk_dtype(TA) !== nothing &&
           ndims(R) <= ndims(A)
            # with init === nothing the reference combines with R's own contents, which must already be the
            # neutral element (mapreduce.jl:161-164): overwriting R gives the same result
            Rn = ndims(R) < ndims(A) ? reshape(R, Base.fill_to_length(size(R), 1, Val(ndims(A)))) : R
            native_mapreducedim!(f, op, Rn, A, init) && return R
        elseif rk_op(op) !== nothing && rk_dtype(TR) !== nothing && rk_dtype(TA) !== nothing && ndims(R) <= ndims(A)
            # f is a closure: mapreduce(x -> x + 1, +, A), count(isodd, A), ...
            Rn = ndims(R) < ndims(A) ? reshape(R, Base.fill_to_length(size(R), 1, Val(ndims(A)))) : R
            native_mapreducedim_closure!(f, op, Rn, A, init) && return R
        end
        return invoke(GPUArrays.mapreducedim!, Tuple{F,OP,AnyROCArray{TR},Union{AbstractArray,Broadcasted}}, f, op, R, A; init)
    end
    # at least one side a wrapper (the dense pair above is more specific)
    @eval function GPUArrays.mapreducedim!(f::F, op::OP, R::ROCStrided{TR}, A::ROCStrided{TA}; init=nothing) where {F,OP,TR,TA}
        if rk_map(f) !== nothing && rk_op(op) !== nothing && rk_dtype(TR) !== nothing && rk_dtype(TA) !== nothing &&
           ndims(R) == ndims(A) && applicable(strides, R) && applicable(strides, A)
            native_mapreducedim_strided!(f, op, R, A, init) && return R
        end
        return invoke(GPUArrays.mapreducedim!, Tuple{F,OP,AnyROCArray{TR},Union{AbstractArray,Broadcasted}}, f, op, R, A; init)
    end
end

# ---- findmax / findmin ----------------------------------------------------------------------------------------
function native_findminmax(wantmax::Bool, A::ROCArray{T,N}, dims) where {T,N}
    mask = UInt32(0)
    for d in (dims === Colon() ? (1:N) : dims)
        d <= N && (mask |= UInt32(1) << (d - 1))
    end
    rdims = ntuple(d -> (mask >> (d - 1)) & 1 == 1 ? 1 : size(A, d), N)
    vals = similar(A, T, rdims)
    idx = similar(A, CartesianIndex{N}, rdims)      # N Int64 per element, the layout the kernel writes
    ws = workspace()
    shape = Int64[size(A)...]
    GC.@preserve A vals idx ws shape begin
        st = ccall((:rk_findminmax, librk[]), Int32,
                   (Int32, Cint, Ptr{Cvoid}, Cint, Ptr{Int64}, UInt32, Ptr{Cvoid}, Ptr{Int64}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                   wantmax, rk_dtype(T), pointer(A), N, shape, mask, pointer(vals),
                   convert(Ptr{Int64}, pointer(idx)), pointer(ws), length(ws), stream_ptr())
    end
    declined(st) && return nothing
    check(st)
    return vals, idx
end
# A a transpose / PermutedDimsArray: the library reduces the parent in memory order and writes the index in the wrapper's
# coordinates; it declines (-> stock method) the dim orders for which the first of equal winners or the output layout
# would differ from the wrapper's column-major order, and views with gaps
function native_findminmax_strided(wantmax::Bool, A::ROCWrapper{T}, dims) where {T}
    N = ndims(A)                 # (not a static parameter: a Transpose does not bind the alias's N)
    mask = UInt32(0)
    for d in (dims === Colon() ? (1:N) : dims)
        d <= N && (mask |= UInt32(1) << (d - 1))
    end
    rdims = ntuple(d -> (mask >> (d - 1)) & 1 == 1 ? 1 : size(A, d), N)
    vals = similar(parent(A), T, rdims)
    idx = similar(parent(A), CartesianIndex{N}, rdims)
    ws = workspace()
    shape = Int64[size(A)...]
    as = strides64(A, N)
    GC.@preserve A vals idx ws shape as begin
        st = ccall((:rk_findminmax_strided, librk[]), Int32,
                   (Int32, Cint, Ptr{Cvoid}, Cint, Ptr{Int64}, Ptr{Int64}, UInt32, Ptr{Cvoid}, Ptr{Int64}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                   wantmax, rk_dtype(T), pointer(A), N, shape, as, mask, pointer(vals),
                   convert(Ptr{Int64}, pointer(idx)), pointer(ws), length(ws), stream_ptr())
    end
    declined(st) && return nothing
    check(st)
    return vals, idx
end
function enable_findminmax!()
    for (fn, wantmax) in ((:findmax, true), (:findmin, false))
        @eval function Base.$fn(A::ROCWrapper{T}; dims=:) where {T<:Union{Float16,Float32,Float64,Int8,Int16,Int32,Int64,UInt16,UInt32,UInt64}}
            N = ndims(A)
            (isempty(A) || !is_strided_wrapper(A)) && return invoke(Base.$fn, Tuple{GPUArrays.AnyGPUArray}, A; dims)
            res = native_findminmax_strided($wantmax, A, dims)
            res === nothing && return invoke(Base.$fn, Tuple{GPUArrays.AnyGPUArray}, A; dims)
            vals, idx = res
            dims === Colon() || return vals, idx
            v = AMDGPU.@allowscalar vals[1]
            i = AMDGPU.@allowscalar idx[1]
            return v, (N == 1 ? i[1] : i)
        end
    end
    for (fn, wantmax) in ((:findmax, true), (:findmin, false))
        @eval function Base.$fn(A::ROCArray{T,N}; dims=:) where {T<:Union{Float16,Float32,Float64,Int8,Int16,Int32,Int64,UInt16,UInt32,UInt64},N}
            isempty(A) && return invoke(Base.$fn, Tuple{GPUArrays.AnyGPUArray}, A; dims)       # the stock method's error
            res = native_findminmax($wantmax, A, dims)
            res === nothing && return invoke(Base.$fn, Tuple{GPUArrays.AnyGPUArray}, A; dims)
            vals, idx = res
            dims === Colon() || return vals, idx
            v = AMDGPU.@allowscalar vals[1]
            i = AMDGPU.@allowscalar idx[1]
            return v, (N == 1 ? i[1] : i)
        end
    end
end

# ---- accumulate -------------------------------------------------------------------------------------------------
function native_accumulate!(op, B::ROCArray{TB,N}, A::ROCArray{TA,N}; init, dims, inclusive::Bool) where {TB,TA,N}
    size(B) == size(A) || throw(DimensionMismatch("accumulate!: $(size(B)) vs $(size(A))"))
    isempty(A) && return true
    dim = dims === nothing ? (N == 1 ? 1 : throw(ArgumentError("accumulate on N-d arrays needs dims"))) : Int(dims)
    shape = Int64[size(A)...]
    need = ccall((:rk_workspace_bytes, librk[]), Csize_t, (Cint, Cint, Cint, Ptr{Int64}, UInt32),
                 2, rk_dtype(TB), N, shape, dim <= N ? UInt32(1) << (dim - 1) : UInt32(0))
    ws = workspace(need)
    note_waiting_call()
    initref = Ref(convert(TB, init))
    GC.@preserve A B ws shape initref begin
        st = ccall((:rk_accumulate, librk[]), Int32,
                   (Cint, Cint, Cint, Ptr{Cvoid}, Ptr{Cvoid}, Cint, Ptr{Int64}, Cint, Int32, Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                   rk_op(op), rk_dtype(TA), rk_dtype(TB), pointer(A), pointer(B), N, shape, dim, inclusive,
                   Base.unsafe_convert(Ptr{Cvoid}, initref), pointer(ws), length(ws), stream_ptr())
    end
    declined(st) && return false
    check(st)
    return true
end

function native_accumulate_strided!(op, B::ROCStrided{TB}, A::ROCStrided{TA}; init, dims, inclusive::Bool) where {TB,TA}
    N = ndims(A)                 # (a Transpose does not bind the alias's N)
    ndims(B) == N || throw(DimensionMismatch("accumulate!: $(size(B)) vs $(size(A))"))
    size(B) == size(A) || throw(DimensionMismatch("accumulate!: $(size(B)) vs $(size(A))"))
    isempty(A) && return true
    dim = dims === nothing ? (N == 1 ? 1 : throw(ArgumentError("accumulate on N-d arrays needs dims"))) : Int(dims)
    shape = Int64[size(A)...]
    as, bs = strides64(A, N), strides64(B, N)
    # the library scans the array in its order of dims in memory: size the bookkeeping for that numbering
    order = sortperm(as)
    mdim = dim <= N ? findfirst(==(dim), order) : N + 1
    need = ccall((:rk_workspace_bytes, librk[]), Csize_t, (Cint, Cint, Cint, Ptr{Int64}, UInt32),
                 2, rk_dtype(TB), N, shape[order], mdim <= N ? UInt32(1) << (mdim - 1) : UInt32(0))
    ws = workspace(need)
    note_waiting_call()
    initref = Ref(convert(TB, init))
    GC.@preserve A B ws shape as bs initref begin
        st = ccall((:rk_accumulate_strided, librk[]), Int32,
                   (Cint, Cint, Cint, Ptr{Cvoid}, Ptr{Cvoid}, Cint, Ptr{Int64}, Ptr{Int64}, Ptr{Int64}, Cint, Int32, Ptr{Cvoid},
                    Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                   rk_op(op), rk_dtype(TA), rk_dtype(TB), pointer(A), pointer(B), N, shape, as, bs, dim, inclusive,
                   Base.unsafe_convert(Ptr{Cvoid}, initref), pointer(ws), length(ws), stream_ptr())
    end
    declined(st) && return false
    check(st)
    return true
end

# 1- and 2-byte element types (Int8, UInt8, Int16, UInt16, Float16) go through the same call: the library scans them in
# the next wider type and stores them narrow (integers wrap like the narrow type itself; Float16 is rounded once, at
# the store, where AcceleratedKernels rounds after every step).
function enable_accumulate!()
    @eval function Base.accumulate!(op, B::ROCArray, A::ROCArray; init=zero(eltype(A)), dims=nothing, inclusive::Bool=true, kwargs...)
        if isempty(kwargs) && rk_op(op) !== nothing && rk_dtype(eltype(A)) !== nothing && rk_dtype(eltype(B)) !== nothing
            native_accumulate!(op, B, A; init, dims, inclusive) && return B
        end
        return AMDGPU.AK.accumulate!(op, B, A, AMDGPU.ROCBackend(); init, dims, inclusive, kwargs...)
    end
    @eval function Base.accumulate!(op, B::ROCStrided, A::ROCStrided; init=zero(eltype(A)), dims=nothing, inclusive::Bool=true, kwargs...)
        if isempty(kwargs) && rk_op(op) !== nothing && rk_dtype(eltype(A)) !== nothing && rk_dtype(eltype(B)) !== nothing &&
           applicable(strides, A) && applicable(strides, B)
            native_accumulate_strided!(op, B, A; init, dims, inclusive) && return B
        end
        return AMDGPU.AK.accumulate!(op, B, A, AMDGPU.ROCBackend(); init, dims, inclusive, kwargs...)
    end
    @eval function Base.accumulate(op, A::ROCArray; init=zero(eltype(A)), kwargs...)
        B = similar(A, Base.promote_op(op, eltype(A), typeof(init)))
        return accumulate!(op, B, A; init, kwargs...)
    end
    @eval Base.cumsum(A::ROCArray; kwargs...) = accumulate(+, A; kwargs...)
    @eval Base.cumprod(A::ROCArray; kwargs...) = accumulate(*, A; init=one(eltype(A)), kwargs...)
end

# ---- fused broadcast: flatten the Broadcasted tree into the postfix program of rk_broadcast -----------------------
const RK_MAX_DIMS, RK_MAX_OPERANDS, RK_MAX_PROGRAM = 8, 8, 48
struct RkOperand
    ptr::Ptr{Cvoid}; dtype::Int32; ndim::Int32; shape::NTuple{8,Int64}; scalar_f::Float64; scalar_i::Int64
    strided::Int32; reserved::Int32; strides::NTuple{8,Int64}
end
const INT_SAFE = (Int32(32), Int32(33), Int32(34), Int32(36), Int32(37), Int32(39), Int32(64), Int32(65), Int32(66), Int32(74),
                  Int32.(96:103)..., Int32(112), Int32.(128:131)...)     # + comparisons, & |, ifelse, ! isodd iseven isnan
# comparisons, max and min of 32-bit intermediates need RK_BC_WRAP_I32 (132) first; this binding keeps such programs
# (an order-sensitive token over a non-leaf Int32 / UInt32 argument) on the stock path instead of typing the tree
const ORDER_SENSITIVE = (Int32(36), Int32(37), Int32.(96:103)..., Int32(128))
struct RkProgram
    compute::Int32; n_operands::Int32; operands::NTuple{8,RkOperand}; n_tokens::Int32; tokens::NTuple{48,Int32}
end
const BINARY = IdDict{Any,Int32}(+ => 32, - => 33, * => 34, / => 35, max => 36, min => 37, ^ => 38,
                                 < => 96, <= => 97, > => 98, >= => 99, == => 100, != => 101, & => 102, | => 103)
const UNARY = IdDict{Any,Int32}(abs => 65, abs2 => 66, sqrt => 67, exp => 68, log => 69, sin => 70, cos => 71,
                                tanh => 72, inv => 73, identity => 74, ! => 128, isodd => 129, iseven => 130, isnan => 131)
struct Unsupported <: Exception end

# Julia computes Float16 arithmetic in Float32 and rounds every result; a Float16 tree runs as a Float32 program with
# RK_BC_ROUND_F16 (134) after every operation whose eltype is Float16
rounds_f16(f) = f in (+, -, *, /, ^, muladd, abs2, sqrt, exp, log, sin, cos, tanh, inv)
function flatten!(ops::Vector{Any}, toks::Vector{Int32}, x)
    if x isa Broadcasted
        flatten_node!(ops, toks, x)
        Broadcast.combine_eltypes(x.f, x.args) === Float16 && rounds_f16(x.f) && push!(toks, Int32(134))
    else
        flatten_node!(ops, toks, x)
    end
end
function flatten_node!(ops::Vector{Any}, toks::Vector{Int32}, x)
    if x isa Broadcasted
        f, args = x.f, x.args
        if length(args) == 1 && f === (-)
            flatten!(ops, toks, args[1]); push!(toks, Int32(64))
        elseif length(args) == 1 && haskey(UNARY, f)
            flatten!(ops, toks, args[1]); push!(toks, UNARY[f])
        elseif length(args) == 2 && haskey(BINARY, f)
            flatten!(ops, toks, args[1]); flatten!(ops, toks, args[2]); push!(toks, BINARY[f])
        elseif length(args) == 3 && f === muladd
            foreach(a -> flatten!(ops, toks, a), args); push!(toks, Int32(39))
        elseif length(args) == 3 && f === ifelse
            foreach(a -> flatten!(ops, toks, a), args); push!(toks, Int32(112))
        elseif f === Base.literal_pow && args[3] isa Val{2}          # x .^ 2
            flatten!(ops, toks, args[2]); push!(toks, Int32(66))
        else
            throw(Unsupported())
        end
    elseif x isa ROCArray || is_strided_wrapper(x) || x isa Union{Float16,Float32,Float64,Int32,Int64,Bool}
        k = findfirst(o -> o === x, ops)
        k === nothing && (push!(ops, x); k = length(ops))
        k > RK_MAX_OPERANDS && throw(Unsupported())
        push!(toks, Int32(k - 1))
    elseif x isa Base.RefValue && x[] isa Number                    # Ref(scalar)
        flatten!(ops, toks, x[])
    else
        throw(Unsupported())                                        # non-strided wrappers, closures, ...
    end
end

function native_copyto!(dest::Union{ROCArray{TD},ROCWrapper{TD}}, bc::Broadcasted) where {TD}
    N = ndims(dest)              # (a Transpose does not bind the alias's N)
    ops, toks = Any[], Int32[]
    flatten!(ops, toks, bc)
    length(toks) <= RK_MAX_PROGRAM || throw(Unsupported())
    CT = promote_type(map(o -> o isa AbstractArray ? eltype(o) : typeof(o), ops)...)
    CT === Float16 && (CT = Float32)
    if !(CT <: Union{Float32,Float64})
        # integer programs of + - * max min muladd - abs abs2 compute in Int64 (the store keeps the low bits);
        # with `/` or a math function Julia's result is a Float64 and so is the compute type
        CT = all(t -> t < RK_MAX_OPERANDS || t in INT_SAFE, toks) && CT <: Union{Bool,Int8,Int16,Int32,Int64,UInt8,UInt16,UInt32} ? Int64 : Float64
        if CT === Int64 && any(t -> t in ORDER_SENSITIVE, toks) &&
           any(o -> (o isa AbstractArray ? eltype(o) : typeof(o)) <: Union{Int8,Int16,Int32,UInt8,UInt16,UInt32}, ops) && count(t -> t >= RK_MAX_OPERANDS, toks) > 1
            throw(Unsupported())                 # would need RK_BC_WRAP_* after the narrow intermediates
        end
    end
    zeros8 = ntuple(_ -> Int64(0), 8)
    zero_op = RkOperand(C_NULL, 0, 0, zeros8, 0.0, 0, 0, 0, zeros8)
    operands = ntuple(RK_MAX_OPERANDS) do k
        k > length(ops) && return zero_op
        o = ops[k]
        if o isa AbstractArray
            rk_dtype(eltype(o)) === nothing && throw(Unsupported())
            shape = ntuple(d -> d <= ndims(o) ? Int64(size(o, d)) : Int64(0), 8)
            if o isa ROCArray
                RkOperand(pointer(o), rk_dtype(eltype(o)), ndims(o), shape, 0.0, 0, 0, 0, zeros8)
            else                                                     # SubArray / Transpose / PermutedDimsArray
                st = strides(o)
                RkOperand(pointer(o), rk_dtype(eltype(o)), ndims(o), shape, 0.0, 0, 1, 0, ntuple(d -> d <= ndims(o) ? Int64(st[d]) : Int64(0), 8))
            end
        else
            RkOperand(C_NULL, rk_dtype(typeof(o)), 0, zeros8, Float64(o), o isa AbstractFloat ? 0 : Int64(o), 0, 0, zeros8)
        end
    end
    prog = Ref(RkProgram(rk_dtype(CT), length(ops), operands, length(toks),
                         ntuple(i -> i <= length(toks) ? toks[i] : Int32(0), 48)))
    shape = Int64[size(dest)...]
    dstrides = dest isa ROCArray ? C_NULL : Int64[strides(dest)...]     # NULL = dense
    GC.@preserve dest ops prog shape dstrides begin
        st = ccall((:rk_broadcast_strided, librk[]), Int32,
                   (Ptr{RkProgram}, Ptr{Cvoid}, Cint, Cint, Ptr{Int64}, Ptr{Int64}, Ptr{Cvoid}),
                   prog, pointer(dest), rk_dtype(TD), N, shape, dstrides, stream_ptr())
    end
    declined(st) && throw(Unsupported())
    check(st)
    return dest
end

function enable_broadcast!()
    @eval function Base.copyto!(dest::Union{ROCArray{TD},ROCWrapper{TD}}, bc::Broadcasted{<:ROCArrayStyle}) where {TD}
        axes(dest) == axes(bc) || Broadcast.throwdm(axes(dest), axes(bc))
        isempty(dest) && return dest
        if rk_dtype(TD) !== nothing && (dest isa ROCArray || is_strided_wrapper(dest))
            try
                return native_copyto!(dest, bc)
            catch e
                e isa Unsupported || rethrow()
            end
        end
        return invoke(Base.copyto!, Tuple{AnyROCArray,Broadcasted{<:GPUArrays.AbstractGPUArrayStyle}}, dest, bc)
    end
end

# ---- volumerhs -----------------------------------------------------------------------------------------------------
"""
    volumerhs!(rhs, Q, vgeo, gravity, D, nelem)

Drop-in for `@roc groupsize=(5,5) gridsize=nelem volumerhs!(rhs, Q, vgeo, gravity, D, nelem)` (perf/volumerhs.jl:200-201).
"""
function volumerhs!(rhs::ROCArray{Float32,5}, Q::ROCArray{Float32,5}, vgeo::ROCArray{Float32,5}, gravity, D::ROCArray{Float32,2}, nelem)
    size(Q) == size(rhs) == (5, 5, 5, 5, nelem) && size(vgeo) == (5, 5, 5, 14, nelem) && size(D) == (5, 5) ||
        throw(DimensionMismatch("volumerhs!: N = 4 layouts expected"))
    GC.@preserve rhs Q vgeo D begin
        check(ccall((:rk_volumerhs_f32, librk[]), Int32,
                    (Ptr{Float32}, Ptr{Float32}, Ptr{Float32}, Float32, Ptr{Float32}, Int64, Ptr{Cvoid}),
                    pointer(rhs), pointer(Q), pointer(vgeo), Float32(gravity), pointer(D), nelem, stream_ptr()))
    end
    return nothing
end

# ---- findall: count, then one stream-compaction pass (replaces src/kernels/indexing.jl:8-36) ---------------------------
function enable_findall!()
    @eval function Base.findall(bools::ROCArray{Bool,N}) where {N}
        I = keytype(bools)
        n = length(bools)
        n == 0 && return ROCArray{I}(undef, 0)
        cnt = sum(reshape(bools, n))                                 # Bool -> Int64 reduction (rk_mapreduce), scalar fetch
        ys = ROCArray{I}(undef, cnt)
        if cnt > 0
            shape = Int64[size(bools)...]
            need = ccall((:rk_workspace_bytes, librk[]), Csize_t, (Cint, Cint, Cint, Ptr{Int64}, UInt32),
                         3, rk_dtype(Bool), N, shape, UInt32(0))     # 3 = RK_KIND_FINDALL
            ws = workspace(need)
            GC.@preserve bools ys shape ws begin
                check(ccall((:rk_findall, librk[]), Int32,
                            (Ptr{UInt8}, Cint, Ptr{Int64}, Ptr{Int64}, Ptr{Int64}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                            convert(Ptr{UInt8}, pointer(bools)), N, shape, convert(Ptr{Int64}, pointer(ys)), C_NULL,
                            pointer(ws), sizeof(ws), stream_ptr()))
            end
        end
        return ys
    end
end

# ---- reverse / reverse! (src/kernels/reverse.jl:59-122): both `_reverse!` kernels -----------------------------------
function enable_reverse!()
    @eval function AMDGPU._reverse!(y::ROCArray{T,N}, x::ROCArray{T,N}; dims=1:ndims(x)) where {T,N}
        size(x) == size(y) || throw(DimensionMismatch("Input and output arrays must equal in size"))
        native_reverse!(y, x, dims) || invoke(AMDGPU._reverse!, Tuple{AMDGPU.AnyROCArray{T,N},AMDGPU.AnyROCArray{T,N}}, y, x; dims)
        return y
    end
    @eval function AMDGPU._reverse!(x::ROCArray{T,N}; dims=1:ndims(x)) where {T,N}
        native_reverse!(x, x, dims) || invoke(AMDGPU._reverse!, Tuple{AMDGPU.AnyROCArray{T,N}}, x; dims)
        return x
    end
end

function native_reverse!(y::ROCArray{T,N}, x::ROCArray{T,N}, dims) where {T,N}
    (isbitstype(T) && sizeof(T) in (1, 2, 4, 8, 16)) || return false
    isempty(x) && return true
    mask = UInt32(0)
    for d in dims
        mask |= UInt32(1) << (d - 1)
    end
    shape = Int64[size(x)...]
    GC.@preserve x y shape begin
        st = ccall((:rk_reverse, librk[]), Int32, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Cint, Ptr{Int64}, UInt32, Ptr{Cvoid}),
                   pointer(x), pointer(y), sizeof(T), N, shape, mask, stream_ptr())
    end
    declined(st) && return false
    check(st)
    return true
end

# ---- permutedims! (GPUArrays' generic kernel in the reference; perf/array.jl:151-155) ----------------------------------
function enable_permutedims!()
    @eval function Base.permutedims!(dest::ROCArray{T,N}, src::ROCArray{T,N}, perm) where {T,N}
        Base.checkdims_perm(axes(dest), axes(src), perm)
        (isbitstype(T) && sizeof(T) in (1, 2, 4, 8, 16)) ||
            return invoke(Base.permutedims!, Tuple{AMDGPU.AnyROCArray,AMDGPU.AnyROCArray,Any}, dest, src, perm)
        isempty(src) && return dest
        shape = Int64[size(src)...]
        p = Int32[perm...]
        GC.@preserve dest src shape p begin
            st = ccall((:rk_permutedims, librk[]), Int32, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Cint, Ptr{Int64}, Ptr{Int32}, Ptr{Cvoid}),
                       pointer(src), pointer(dest), sizeof(T), N, shape, p, stream_ptr())
        end
        declined(st) && return invoke(Base.permutedims!, Tuple{AMDGPU.AnyROCArray,AMDGPU.AnyROCArray,Any}, dest, src, perm)
        check(st)
        return dest
    end
end

# ---- sort! / sortperm! (src/kernels/sorting.jl:1-3) ----------------------------------------------------------------------
# Native: the default order, `rev`, `lt = !isless` (the descending order: test/hip_rocarray/sorting.jl:20-22) and any `by`
# whose keys `by.(x)` have a sortable eltype (:24-26): map (the fused broadcast), sortperm of the keys, gather.  Any other
# `lt` stays with AcceleratedKernels.
const SORTABLE = Union{Float16,Float32,Float64,Int16,Int32,Int64}
# false / true: `lt` is isless / !isless (reverses the order); nothing: a comparator the library has no form for
native_order(lt) = lt === isless ? false : (lt isa ComposedFunction{typeof(!),typeof(isless)} ? true : nothing)

function enable_sort!()
    @eval function Base.sort!(x::ROCVector{T}; rev::Bool=false, lt=isless, by=identity, kwargs...) where {T<:SORTABLE}
        flip = native_order(lt)
        (flip !== nothing && isempty(kwargs)) || return (AMDGPU.AK.sort!(x; rev, lt, by, kwargs...); x)
        rev = xor(rev, flip)
        n = length(x)
        n > 1 || return x
        if by !== identity
            keys = by.(x)
            eltype(keys) <: SORTABLE || return (AMDGPU.AK.sort!(x; rev, by, kwargs...); x)
            p = sortperm(keys; rev)
            copyto!(x, x[p])
            AMDGPU.unsafe_free!(keys); AMDGPU.unsafe_free!(p)
            return x
        end
        tmp = ROCVector{UInt8}(undef, ccall((:rk_sort_tmp_bytes, librk[]), Csize_t, (Cint, Int64, Int32), rk_dtype(T), n, 0))
        GC.@preserve x tmp begin
            st = ccall((:rk_sort, librk[]), Int32, (Cint, Ptr{Cvoid}, Int64, Int32, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                       rk_dtype(T), pointer(x), n, rev, pointer(tmp), sizeof(tmp), stream_ptr())
        end
        note_sort(tmp, n)                                           # freed at once, or kept until its record has been read
        declined(st) && return (AMDGPU.AK.sort!(x; rev); x)          # rk_sort validates before it writes
        check(st)
        return x
    end
    @eval function Base.sortperm!(ix::ROCVector{Int}, x::ROCVector{T}; rev::Bool=false, lt=isless, by=identity, kwargs...) where {T<:SORTABLE}
        flip = native_order(lt)
        (flip !== nothing && isempty(kwargs)) || return (AMDGPU.AK.sortperm!(ix, x; rev, lt, by, kwargs...); ix)
        rev = xor(rev, flip)
        if by !== identity
            keys = by.(x)
            eltype(keys) <: SORTABLE || return (AMDGPU.AK.sortperm!(ix, x; rev, by, kwargs...); ix)
            return sortperm!(ix, keys; rev)
        end
        n = length(x)
        length(ix) == n || throw(DimensionMismatch("sortperm!: index vector of length $(length(ix)) for $n keys"))
        n > 0 || return ix
        tmp = ROCVector{UInt8}(undef, ccall((:rk_sort_tmp_bytes, librk[]), Csize_t, (Cint, Int64, Int32), rk_dtype(T), n, 1))
        GC.@preserve ix x tmp begin
            st = ccall((:rk_sortperm, librk[]), Int32, (Cint, Ptr{Cvoid}, Ptr{Int64}, Int64, Int32, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                       rk_dtype(T), pointer(x), pointer(ix), n, rev, pointer(tmp), sizeof(tmp), stream_ptr())
        end
        note_sort(tmp, n)
        declined(st) && return (AMDGPU.AK.sortperm!(ix, x; rev); ix)
        check(st)
        return ix
    end
end

"""
    enable!()

Install the native methods.  Call once after `using AMDGPU`.
"""
function enable!()
    isfile(librk[]) || error("librk.so not found at $(librk[]); build it with `python amdgpu.jl_amd/build.py`")
    ccall((:rk_version, librk[]), Int32, ()) >= 100 || error("librk.so is too old")
    enable_mapreduce!(); enable_findminmax!(); enable_accumulate!(); enable_broadcast!(); enable_findall!(); enable_reverse!(); enable_permutedims!(); enable_sort!(); enable_wait_checks!()
    return nothing
end

end # module
