# MIWMMA.jl -- Julia host side of the MI355X WMMA / GEMM path.
#
# Keeps the call surface of CUDAnative.jl for this path and reaches the HIP kernels through
# `ccall` into the prebuilt libmiwmma.so (C ABI: include/miwmma.h):
#
#   CUDAnative.jl                                      here
#   ------------------------------------------------   -----------------------------------------
#   CuHostArray            src/array.jl:4-70            MIWMMA.DeviceBuffer (hipMalloc-backed)
#   DevicePtr{T,AS}, AS    src/device/pointer.jl:11-109 MIWMMA.DevicePtr{T,A}, MIWMMA.AS
#   WMMA.Config/Fragment/load_a/load_b/load_c/mma/
#   store_d/fill_c, f.(frag, s)  src/device/cuda/wmma.jl:300-716   MIWMMA.WMMA.*
#   @cuda threads=.. f(args...)  src/execution.jl:45-114           MIWMMA.@hip threads=64 f(args...)
#
# In CUDAnative the WMMA functions are device functions that a JIT-compiled kernel calls from 32
# lanes.  There is no Julia->GPU compiler here: the kernels are compiled ahead of time, every
# fragment operation is one launch of a 64-lane wavefront, and a Fragment that comes from memory
# is a device-resident image of the wavefront's registers (64 lanes x 4 elements).  A kernel
# function written with WMMA.load_a ... WMMA.store_d therefore reads exactly like
# examples/wmma/high-level.jl and runs on the GPU when called through @hip.
#
# This file has not been executed in the build environment of this repository (no Julia there);
# the same C ABI is exercised by the Python mirror and its tests.  Needs Julia >= 1.6.

module MIWMMA

export DeviceBuffer, DevicePtr, AS, WMMA, @hip, gemm!, synchronize, MIWError

const libmiwmma = get(ENV, "MIWMMA_LIB", joinpath(@__DIR__, "..", "libmiwmma.so"))

# ---------------------------------------------------------------------------- errors ------

struct MIWError <: Exception
    code::Cint
    msg::String
end
Base.showerror(io::IO, e::MIWError) = print(io, "miwmma error ", e.code, ": ", e.msg)

last_error() = unsafe_string(ccall((:miw_last_error, libmiwmma), Cstring, ()))
check(rc::Cint) = rc == 0 ? nothing : throw(MIWError(rc, last_error()))

const hipErrorOutOfMemory = Cint(2)

function init(device::Integer=0)
    check(ccall((:miw_init, libmiwmma), Cint, (Cint,), device))
end

synchronize(stream::Ptr{Cvoid}=C_NULL) = check(ccall((:miw_sync, libmiwmma), Cint, (Ptr{Cvoid},), stream))

# ---------------------------------------------------------------------------- memory ------

module AS
    abstract type AddressSpace end
    struct Generic  <: AddressSpace end
    struct Global   <: AddressSpace end
    struct Shared   <: AddressSpace end
    struct Constant <: AddressSpace end
    struct Local    <: AddressSpace end
end
as_code(::Type{AS.Generic}) = Cint(0)
as_code(::Type{AS.Global})  = Cint(1)
as_code(::Type{AS.Shared})  = Cint(3)
as_code(::Type{A}) where {A} = error("Invalid address space for WMMA: $A")

"Typed device address with an address-space tag (src/device/pointer.jl:46-55)."
struct DevicePtr{T,A}
    addr::UInt
end
Base.eltype(::Type{<:DevicePtr{T}}) where {T} = T
Base.:(+)(p::DevicePtr{T,A}, n::Integer) where {T,A} = DevicePtr{T,A}(p.addr + UInt(n))
Base.:(==)(a::DevicePtr{T,A}, b::DevicePtr{U,B}) where {T,A,U,B} = a.addr == b.addr && A == B

"hipMalloc-backed array (pointer, dims); the CuHostArray of src/array.jl."
mutable struct DeviceBuffer{T,N}
    ptr::Ptr{Cvoid}
    dims::Dims{N}
end

function DeviceBuffer{T,N}(::UndefInitializer, dims::Dims{N}) where {T,N}
    sz = prod(dims) * sizeof(T)
    p = Ref{Ptr{Cvoid}}(C_NULL)
    rc = ccall((:miw_malloc, libmiwmma), Cint, (Ptr{Ptr{Cvoid}}, Csize_t), p, sz)
    if rc == hipErrorOutOfMemory
        GC.gc(true)                       # src/array.jl:23-29: collect, then retry once
        rc = ccall((:miw_malloc, libmiwmma), Cint, (Ptr{Ptr{Cvoid}}, Csize_t), p, sz)
    end
    check(rc)
    obj = DeviceBuffer{T,N}(p[], dims)
    finalizer(obj) do a
        a.ptr == C_NULL || ccall((:miw_free, libmiwmma), Cint, (Ptr{Cvoid},), a.ptr)
        a.ptr = C_NULL
    end
    return obj
end
DeviceBuffer{T}(::UndefInitializer, dims::Integer...) where {T} = DeviceBuffer{T,length(dims)}(undef, Dims(dims))

function DeviceBuffer(src::Array{T,N}) where {T,N}
    dst = DeviceBuffer{T,N}(undef, size(src))
    GC.@preserve src check(ccall((:miw_memcpy_h2d, libmiwmma), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t),
                                 dst.ptr, pointer(src), sizeof(src)))
    return dst
end

function Base.Array(src::DeviceBuffer{T,N}) where {T,N}
    dst = Array{T,N}(undef, src.dims)
    GC.@preserve dst check(ccall((:miw_memcpy_d2h, libmiwmma), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t),
                                 pointer(dst), src.ptr, sizeof(dst)))
    return dst
end

Base.size(a::DeviceBuffer) = a.dims
Base.length(a::DeviceBuffer) = prod(a.dims)
Base.similar(a::DeviceBuffer{T,N}) where {T,N} = DeviceBuffer{T,N}(undef, a.dims)
Base.pointer(a::DeviceBuffer{T}, i::Integer=1) where {T} =
    DevicePtr{T,AS.Global}(UInt(a.ptr) + UInt((i - 1) * sizeof(T)))

# ---------------------------------------------------------------------------- WMMA --------

module WMMA

using ..MIWMMA: libmiwmma, check, DevicePtr, DeviceBuffer, AS, as_code

export FragmentLayout, RowMajor, ColMajor, Unspecified, MatrixA, MatrixB, Accumulator,
       Fragment, Config, load_a, load_b, load_c, mma, store_d, fill_c

abstract type FragmentLayout end
struct RowMajor <: FragmentLayout end
struct ColMajor <: FragmentLayout end
struct Unspecified <: FragmentLayout end

abstract type FragmentUse end
struct MatrixA <: FragmentUse end
struct MatrixB <: FragmentUse end
struct Accumulator <: FragmentUse end

struct Config{M, N, K, d_type} end

const WAVEFRONT = 64
const FS = 4            # elements per lane of every 16x16x16 fragment on wave64

"""
Fragment{M,N,K,FS,T,L,U}: `x` is the device-resident image of the wavefront's registers
(element i of lane l at index l*FS + i); the order of elements is unspecified.
"""
struct Fragment{M, N, K, FS, T, L <: FragmentLayout, U <: FragmentUse}
    x::DeviceBuffer{T,2}
end

const stream = Ref{Ptr{Cvoid}}(C_NULL)   # set by @hip stream=...

dtype_code(::Type{Float16}) = Cint(0)
dtype_code(::Type{Float32}) = Cint(1)
dtype_code(::Type{T}) where {T} = error("Invalid element type for WMMA: $T")
layout_code(::Type{RowMajor}) = Cint(0)
layout_code(::Type{ColMajor}) = Cint(1)
layout_code(::Type{L}) where {L} = error("Invalid layout for WMMA: $L")
use_code(::Type{MatrixA}) = Cint(0)
use_code(::Type{MatrixB}) = Cint(1)
use_code(::Type{Accumulator}) = Cint(2)
check_shape(M, N, K) = (M, N, K) == (16, 16, 16) || error("Invalid shape for WMMA: (M, N, K) = ($M, $N, $K)")

for (mat, U) in (("a", MatrixA), ("b", MatrixB), ("c", Accumulator))
    fname = Symbol("load_$mat")
    @eval function $fname(addr::DevicePtr{T, A}, stride::Number, layout::Type{L},
                          config::Type{Config{M, N, K, D}}) where {T, A, L, M, N, K, D}
        check_shape(M, N, K)
        $(mat != "c") && T !== Float16 && error("Invalid type $T for matrix $($mat)")
        L_ret = $(mat == "c") ? Unspecified : L
        img = DeviceBuffer{T,2}(undef, (FS, WAVEFRONT))
        check(ccall((:miw_frag_load, libmiwmma), Cint,
                    (Cint, Cint, Cint, Cint, Cint, Cint, Cint, Ptr{Cvoid}, Int64, Ptr{Cvoid}, Ptr{Cvoid}),
                    use_code($U), dtype_code(T), layout_code(L), as_code(A), M, N, K,
                    Ptr{Cvoid}(addr.addr), Int64(stride), img.ptr, stream[]))
        return Fragment{M, N, K, FS, T, L_ret, $U}(img)
    end
end

function fill_c(value::T, config::Type{Config{M, N, K, D}}) where {T, M, N, K, D}
    check_shape(M, N, K)
    img = DeviceBuffer{T,2}(undef, (FS, WAVEFRONT))
    check(ccall((:miw_frag_fill, libmiwmma), Cint, (Cint, Cfloat, Ptr{Cvoid}, Ptr{Cvoid}),
                dtype_code(T), Float32(value), img.ptr, stream[]))
    return Fragment{M, N, K, FS, T, Unspecified, Accumulator}(img)
end

function mma(a::Fragment{M, N, K, A_SZ, A_T, A_L, MatrixA},
             b::Fragment{M, N, K, B_SZ, B_T, B_L, MatrixB},
             c::Fragment{M, N, K, C_SZ, C_T, Unspecified, Accumulator},
             config::Type{Config{M, N, K, D_T}}) where {M, N, K, A_SZ, A_T, A_L, B_SZ, B_T, B_L, C_SZ, C_T, D_T}
    check_shape(M, N, K)
    img = DeviceBuffer{D_T,2}(undef, (FS, WAVEFRONT))
    check(ccall((:miw_frag_mma, libmiwmma), Cint,
                (Cint, Cint, Cint, Cint, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
                layout_code(A_L), layout_code(B_L), dtype_code(C_T), dtype_code(D_T),
                a.x.ptr, b.x.ptr, c.x.ptr, img.ptr, stream[]))
    return Fragment{M, N, K, FS, D_T, Unspecified, Accumulator}(img)
end

function store_d(addr::DevicePtr{T, A}, d::Fragment{M, N, K, D_SZ, T, Unspecified, Accumulator},
                 stride::Number, layout::Type{L}, config::Type{Config{M, N, K, T}}) where {T, A, M, N, K, D_SZ, L}
    check_shape(M, N, K)
    check(ccall((:miw_frag_store, libmiwmma), Cint,
                (Cint, Cint, Cint, Cint, Cint, Cint, Ptr{Cvoid}, Ptr{Cvoid}, Int64, Ptr{Cvoid}),
                dtype_code(T), layout_code(L), as_code(A), M, N, K,
                Ptr{Cvoid}(addr.addr), d.x.ptr, Int64(stride), stream[]))
    return nothing
end

# f.(frag, scalar): .* and .+ keep the Fragment type (src/device/cuda/wmma.jl:678-716)
struct FragmentBroadcastStyle <: Broadcast.BroadcastStyle end
Base.BroadcastStyle(::Type{<:Fragment}) = FragmentBroadcastStyle()
Base.BroadcastStyle(s::FragmentBroadcastStyle, ::Broadcast.DefaultArrayStyle{0}) = s
Base.broadcastable(frag::Fragment) = frag
Base.axes(frag::Fragment) = (Base.OneTo(FS),)

function frag_map(op::Cint, s::Number, f::Fragment{M, N, K, FSZ, T, L, U}) where {M, N, K, FSZ, T, L, U}
    img = DeviceBuffer{T,2}(undef, (FS, WAVEFRONT))
    check(ccall((:miw_frag_map, libmiwmma), Cint, (Cint, Cint, Cfloat, Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                dtype_code(T), op, Float32(T(s)), f.x.ptr, img.ptr, FS * WAVEFRONT, stream[]))
    return Fragment{M, N, K, FSZ, T, L, U}(img)
end

function Base.copy(bc::Broadcast.Broadcasted{FragmentBroadcastStyle})
    frag = something(filter(a -> a isa Fragment, collect(Any, bc.args))...)
    scal = filter(a -> !(a isa Fragment), collect(Any, bc.args))
    length(scal) == 1 || throw(DimensionMismatch("WMMA fragment broadcast takes one fragment and one scalar"))
    s = scal[1] isa Ref ? scal[1][] : scal[1]
    bc.f === (*) && return frag_map(Cint(0), s, frag)
    bc.f === (+) && return frag_map(Cint(1), s, frag)
    error("only .* and .+ are available on device fragments")
end

end # module WMMA

# ---------------------------------------------------------------------------- launch ------

"""
    @hip threads=64 [stream=s] kernel(args...)

The `@cuda` of src/execution.jl:45-114 for kernels written with the WMMA fragment operations:
runs `kernel(args...)` with one wavefront (threads must be 64, blocks 1); every fragment operation
inside is a device launch on `stream`.  Arguments are kept alive until the call returns.
"""
macro hip(ex...)
    call = ex[end]
    Meta.isexpr(call, :call) || throw(ArgumentError("second argument to @hip should be a function call"))
    threads, blocks, strm = 64, 1, :(C_NULL)
    for kw in ex[1:end-1]
        Meta.isexpr(kw, :(=)) || throw(ArgumentError("expected keyword arguments before the call"))
        key, val = kw.args
        if key == :threads
            threads = val
        elseif key == :blocks
            blocks = val
        elseif key == :stream
            strm = val
        elseif key in (:shmem, :config)
            # accepted for source compatibility; a fragment kernel has no launch-time LDS or occupancy choice
        else
            throw(ArgumentError("Unsupported keyword argument '$key'"))
        end
    end
    f, args = call.args[1], call.args[2:end]
    quote
        ($(esc(threads)) == 64 && $(esc(blocks)) == 1) ||
            throw(MIWError(Cint(-1), "a WMMA fragment kernel runs as one wavefront: threads=64, blocks=1"))
        local old = WMMA.stream[]
        WMMA.stream[] = $(esc(strm))
        try
            GC.@preserve $(map(esc, args)...) $(esc(f))($(map(esc, args)...))
        finally
            WMMA.stream[] = old
        end
    end
end

# ---------------------------------------------------------------------------- GEMM --------

struct GemmDesc
    m::Int64; n::Int64; k::Int64
    lda::Int64; ldb::Int64; ldc::Int64; ldd::Int64
    a_layout::Cint; b_layout::Cint; c_layout::Cint; d_layout::Cint
    c_type::Cint; d_type::Cint
    acc_type::Cint; acc_chunk::Cint
    alpha::Cfloat; beta::Cfloat
    use_c::Cint
    batch::Int64
    stride_a::Int64; stride_b::Int64; stride_c::Int64; stride_d::Int64
    variant::Cint
end

"""
    gemm!(D, A, B, C; alpha=1, beta=1, a_layout=ColMajor, ..., acc_type=Float32, batch=1)

D = alpha*A*B + beta*C on the tiled MFMA kernel (asynchronous; call `synchronize()` before
reading D).  A, B are `DeviceBuffer{Float16}`; C, D `DeviceBuffer{Float16}` or `{Float32}`.
"""
function gemm!(D::DeviceBuffer{DT}, A::DeviceBuffer{Float16}, B::DeviceBuffer{Float16},
               C::Union{DeviceBuffer{CT},Nothing}, M::Integer, N::Integer, K::Integer;
               alpha=1f0, beta=1f0, a_layout=WMMA.ColMajor, b_layout=WMMA.ColMajor,
               c_layout=WMMA.ColMajor, d_layout=WMMA.ColMajor, acc_type=Float32, acc_chunk=0,
               batch=1, variant=0, stream::Ptr{Cvoid}=C_NULL) where {DT, CT}
    cty = C === nothing ? Float32 : CT
    desc = Ref(GemmDesc(M, N, K, 0, 0, 0, 0, WMMA.layout_code(a_layout), WMMA.layout_code(b_layout),
                        WMMA.layout_code(c_layout), WMMA.layout_code(d_layout), WMMA.dtype_code(cty),
                        WMMA.dtype_code(DT), WMMA.dtype_code(acc_type), acc_chunk, alpha, beta,
                        C === nothing ? 0 : 1, batch, 0, 0, 0, 0, variant))
    GC.@preserve A B C D check(ccall((:miw_gemm, libmiwmma), Cint,
        (Ptr{GemmDesc}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        desc, A.ptr, B.ptr, C === nothing ? C_NULL : C.ptr, D.ptr, stream))
    return D
end

end # module MIWMMA

#= Usage, mirroring examples/wmma/high-level.jl:

using .MIWMMA, .MIWMMA.WMMA
MIWMMA.init(0)
a = rand(Float16, (16, 16)); b = rand(Float16, (16, 16)); c = rand(Float32, (16, 16))
a_dev, b_dev, c_dev = DeviceBuffer(a), DeviceBuffer(b), DeviceBuffer(c)
d_dev = similar(c_dev)

function kernel(a_dev, b_dev, c_dev, d_dev)
    conf = WMMA.Config{16, 16, 16, Float32}
    a_frag = WMMA.load_a(pointer(a_dev), 16, WMMA.ColMajor, conf)
    b_frag = WMMA.load_b(pointer(b_dev), 16, WMMA.ColMajor, conf)
    c_frag = WMMA.load_c(pointer(c_dev), 16, WMMA.ColMajor, conf)
    c_frag = 0.5f0 .* c_frag
    d_frag = WMMA.mma(a_frag, b_frag, c_frag, conf)
    WMMA.store_d(pointer(d_dev), d_frag, 16, WMMA.ColMajor, conf)
    return
end

@hip threads=64 kernel(a_dev, b_dev, c_dev, d_dev)
d = Array(d_dev)
@assert all(isapprox.(Float32.(a) * Float32.(b) + 0.5f0 * c, d; rtol=0.01))
=#
