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
#   llvm_wmma_{load,store,mma}_*  src/device/cuda/wmma.jl:104-257  MIWMMA.WMMA.llvm_wmma_* (the same 52 names)
#   flatten / unflatten           src/device/cuda/wmma.jl:264-294  MIWMMA.WMMA.flatten / unflatten
#   @cuda threads=.. f(args...)  src/execution.jl:45-114           MIWMMA.@hip threads=64 f(args...)
#   cufunction / HostKernel, registers/memory/maxthreads, config=  MIWMMA.hipfunction / HostKernel,
#                                 src/execution.jl:205-297          registers/memory/maxthreads, launch_configuration
#   CuModule(image), CuFunction(mod, name)  src/execution.jl:300-342   MIWMMA.CodeObject, kernel(mod, name)
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

export DeviceBuffer, DevicePtr, AS, WMMA, @hip, gemm!, gemm_splitk!, gemm_splitk_static!, synchronize, MIWError,
       HostKernel, hipfunction, CodeObject, kernel, registers, memory, maxthreads, launch_configuration,
       Stream, device_info, warpsize, nextwarp, prevwarp, mem_info

const libmiwmma = get(ENV, "MIWMMA_LIB", joinpath(@__DIR__, "..", "libmiwmma.so"))

# ---------------------------------------------------------------------------- errors ------

struct MIWError <: Exception
    code::Cint
    msg::String
end
Base.showerror(io::IO, e::MIWError) = print(io, "miwmma error ", e.code, ": ", e.msg)

last_error() = unsafe_string(ccall((:miw_last_error, libmiwmma), Cstring, ()))
check(rc::Cint) = rc == 0 ? nothing : throw(MIWError(rc, last_error()))
"Hash of the sources the loaded library was built from."
build_id() = unsafe_string(ccall((:miw_build_id, libmiwmma), Cstring, ()))

const hipErrorOutOfMemory = Cint(2)

function init(device::Integer=0)
    check(ccall((:miw_init, libmiwmma), Cint, (Cint,), device))
end

"Device properties (miw_device_info of include/miwmma.h, field for field)."
struct DeviceInfo
    name::NTuple{128,UInt8}
    arch::NTuple{64,UInt8}
    cu_count::Cint
    wave_size::Cint
    clock_mhz::Cint
    mem_clock_mhz::Cint
    mem_bus_bits::Cint
    l2_bytes::Cint
    max_threads_per_block::Cint
    lds_per_block::Csize_t
    hbm_bytes::Csize_t
    peak_f16_tflops::Cdouble
end
cstring(t::NTuple{N,UInt8}) where {N} = String(collect(Iterators.takewhile(!=(0x00), t)))

function device_info()
    info = Ref{DeviceInfo}()
    check(ccall((:miw_device_info_get, libmiwmma), Cint, (Ptr{DeviceInfo},), info))
    d = info[]
    return (name=cstring(d.name), arch=cstring(d.arch), cu_count=Int(d.cu_count), wave_size=Int(d.wave_size),
            clock_mhz=Int(d.clock_mhz), lds_per_block=Int(d.lds_per_block), hbm_bytes=Int(d.hbm_bytes),
            peak_f16_tflops=d.peak_f16_tflops)
end

"Lanes of a wavefront (CUDAdrv.warpsize): 64 on gfx950.  `dev` is what device_info() returns."
warpsize(dev=device_info()) = dev.wave_size

"""
    nextwarp(dev, threads)
    prevwarp(dev, threads)

The next or previous nearest number of threads that is a multiple of the wavefront size of the
device (src/execution.jl:418-426).
"""
function nextwarp(dev, threads::Integer)
    ws = warpsize(dev)
    return threads + (ws - threads % ws) % ws
end
function prevwarp(dev, threads::Integer)
    ws = warpsize(dev)
    return threads - rem(threads, ws)
end

# ---------------------------------------------------------------------------- streams -----

"A HIP stream (the `stream=` keyword of @cuda, src/execution.jl:59-63)."
mutable struct Stream
    handle::Ptr{Cvoid}
    function Stream()
        p = Ref{Ptr{Cvoid}}(C_NULL)
        check(ccall((:miw_stream_create, libmiwmma), Cint, (Ptr{Ptr{Cvoid}},), p))
        s = new(p[])
        finalizer(s) do x
            x.handle == C_NULL || ccall((:miw_stream_destroy, libmiwmma), Cint, (Ptr{Cvoid},), x.handle)
            x.handle = C_NULL
        end
        return s
    end
end
stream_handle(s::Stream) = s.handle
stream_handle(s::Ptr{Cvoid}) = s
stream_handle(::Nothing) = C_NULL

synchronize(stream=C_NULL) = check(ccall((:miw_sync, libmiwmma), Cint, (Ptr{Cvoid},), stream_handle(stream)))

# The stream fragment operations run on is a property of the running task, as CUDAnative's
# launches from Threads.@threads need (test/device/execution.jl:1057-1076): @hip stream=s sets it
# for the body's task only.
current_stream() = get(task_local_storage(), :miwmma_stream, C_NULL)::Ptr{Cvoid}
with_stream(f, s) = task_local_storage(f, :miwmma_stream, stream_handle(s))

# CuEvent timing as test/perf/launch_overhead uses it
mutable struct Event
    handle::Ptr{Cvoid}
    function Event()
        p = Ref{Ptr{Cvoid}}(C_NULL)
        check(ccall((:miw_event_create, libmiwmma), Cint, (Ptr{Ptr{Cvoid}},), p))
        e = new(p[])
        finalizer(e) do x
            x.handle == C_NULL || ccall((:miw_event_destroy, libmiwmma), Cint, (Ptr{Cvoid},), x.handle)
            x.handle = C_NULL
        end
        return e
    end
end
record(e::Event, stream=C_NULL) = check(ccall((:miw_event_record, libmiwmma), Cint, (Ptr{Cvoid}, Ptr{Cvoid}), e.handle, stream_handle(stream)))
synchronize(e::Event) = check(ccall((:miw_event_synchronize, libmiwmma), Cint, (Ptr{Cvoid},), e.handle))
function elapsed_ms(start::Event, stop::Event)
    ms = Ref{Cfloat}(0)
    check(ccall((:miw_event_elapsed_ms, libmiwmma), Cint, (Ptr{Cfloat}, Ptr{Cvoid}, Ptr{Cvoid}), ms, start.handle, stop.handle))
    return ms[]
end

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

function Base.copyto!(dst::DeviceBuffer{T}, src::DeviceBuffer{T}) where {T}
    length(dst) == length(src) || throw(DimensionMismatch("device copy between buffers of different length"))
    check(ccall((:miw_memcpy_d2d, libmiwmma), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t), dst.ptr, src.ptr, length(src) * sizeof(T)))
    return dst
end
"(free, total) bytes of device memory."
function mem_info()
    f, t = Ref{Csize_t}(0), Ref{Csize_t}(0)
    check(ccall((:miw_mem_info, libmiwmma), Cint, (Ptr{Csize_t}, Ptr{Csize_t}), f, t))
    return Int(f[]), Int(t[])
end

function Base.fill!(a::DeviceBuffer{T}, byte::UInt8) where {T}
    check(ccall((:miw_memset, libmiwmma), Cint, (Ptr{Cvoid}, Cint, Csize_t), a.ptr, byte, length(a) * sizeof(T)))
    return a
end

Base.size(a::DeviceBuffer) = a.dims
Base.length(a::DeviceBuffer) = prod(a.dims)
Base.similar(a::DeviceBuffer{T,N}) where {T,N} = DeviceBuffer{T,N}(undef, a.dims)
Base.pointer(a::DeviceBuffer{T}, i::Integer=1) where {T} =
    DevicePtr{T,AS.Global}(UInt(a.ptr) + UInt((i - 1) * sizeof(T)))

# ---------------------------------------------------------------------------- WMMA --------

module WMMA

using ..MIWMMA: libmiwmma, check, DevicePtr, DeviceBuffer, AS, as_code, current_stream

export FragmentLayout, RowMajor, ColMajor, Unspecified, MatrixA, MatrixB, Accumulator,
       Fragment, Config, load_a, load_b, load_c, mma, store_d, fill_c, flatten, unflatten

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

"Elements per lane and bytes of a fragment image, as the library reports them."
elems_per_lane(::Type{U}, ::Type{T}) where {U, T} =
    Int(ccall((:miw_frag_elems_per_lane, libmiwmma), Cint, (Cint, Cint), use_code(U), dtype_code(T)))
image_bytes(::Type{U}, ::Type{T}) where {U, T} =
    Int(ccall((:miw_frag_image_bytes, libmiwmma), Csize_t, (Cint, Cint), use_code(U), dtype_code(T)))

# One launch that reads a tile into a fresh fragment image.
function load_image(::Type{U}, ::Type{T}, ::Type{L}, ::Type{A}, addr::UInt, stride::Integer) where {U, T, L, A}
    img = DeviceBuffer{T,2}(undef, (FS, WAVEFRONT))
    check(ccall((:miw_frag_load, libmiwmma), Cint,
                (Cint, Cint, Cint, Cint, Cint, Cint, Cint, Ptr{Cvoid}, Int64, Ptr{Cvoid}, Ptr{Cvoid}),
                use_code(U), dtype_code(T), layout_code(L), as_code(A), 16, 16, 16,
                Ptr{Cvoid}(addr), Int64(stride), img.ptr, current_stream()))
    return img
end

for (mat, U) in (("a", MatrixA), ("b", MatrixB), ("c", Accumulator))
    fname = Symbol("load_$mat")
    @eval function $fname(addr::DevicePtr{T, A}, stride::Number, layout::Type{L},
                          config::Type{Config{M, N, K, D}}) where {T, A, L, M, N, K, D}
        check_shape(M, N, K)
        $(mat != "c") && T !== Float16 && error("Invalid type $T for matrix $($mat)")
        L_ret = $(mat == "c") ? Unspecified : L
        return Fragment{M, N, K, FS, T, L_ret, $U}(load_image($U, T, L, A, addr.addr, stride))
    end
end

function fill_image(::Type{T}, value) where {T}
    img = DeviceBuffer{T,2}(undef, (FS, WAVEFRONT))
    check(ccall((:miw_frag_fill, libmiwmma), Cint, (Cint, Cfloat, Ptr{Cvoid}, Ptr{Cvoid}),
                dtype_code(T), Float32(value), img.ptr, current_stream()))
    return img
end

function fill_c(value::T, config::Type{Config{M, N, K, D}}) where {T, M, N, K, D}
    check_shape(M, N, K)
    return Fragment{M, N, K, FS, T, Unspecified, Accumulator}(fill_image(T, value))
end

function mma_image(::Type{LA}, ::Type{LB}, ::Type{CT}, ::Type{DT}, a::DeviceBuffer, b::DeviceBuffer,
                   c::DeviceBuffer) where {LA, LB, CT, DT}
    img = DeviceBuffer{DT,2}(undef, (FS, WAVEFRONT))
    check(ccall((:miw_frag_mma, libmiwmma), Cint,
                (Cint, Cint, Cint, Cint, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
                layout_code(LA), layout_code(LB), dtype_code(CT), dtype_code(DT),
                a.ptr, b.ptr, c.ptr, img.ptr, current_stream()))
    return img
end

function mma(a::Fragment{M, N, K, A_SZ, A_T, A_L, MatrixA},
             b::Fragment{M, N, K, B_SZ, B_T, B_L, MatrixB},
             c::Fragment{M, N, K, C_SZ, C_T, Unspecified, Accumulator},
             config::Type{Config{M, N, K, D_T}}) where {M, N, K, A_SZ, A_T, A_L, B_SZ, B_T, B_L, C_SZ, C_T, D_T}
    check_shape(M, N, K)
    return Fragment{M, N, K, FS, D_T, Unspecified, Accumulator}(mma_image(A_L, B_L, C_T, D_T, a.x, b.x, c.x))
end

function store_image(::Type{T}, ::Type{L}, ::Type{A}, addr::UInt, img::DeviceBuffer, stride::Integer) where {T, L, A}
    check(ccall((:miw_frag_store, libmiwmma), Cint,
                (Cint, Cint, Cint, Cint, Cint, Cint, Ptr{Cvoid}, Ptr{Cvoid}, Int64, Ptr{Cvoid}),
                dtype_code(T), layout_code(L), as_code(A), 16, 16, 16,
                Ptr{Cvoid}(addr), img.ptr, Int64(stride), current_stream()))
    return nothing
end

function store_d(addr::DevicePtr{T, A}, d::Fragment{M, N, K, D_SZ, T, Unspecified, Accumulator},
                 stride::Number, layout::Type{L}, config::Type{Config{M, N, K, T}}) where {T, A, M, N, K, D_SZ, L}
    check_shape(M, N, K)
    return store_image(T, L, A, addr.addr, d.x, stride)
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
                dtype_code(T), op, Float32(T(s)), f.x.ptr, img.ptr, FS * WAVEFRONT, current_stream()))
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

# The whole kernel of examples/wmma/high-level.jl:30-44 fused in one launch (miw_wmma_mac).
struct MacDesc
    m::Cint; n::Cint; k::Cint
    a_layout::Cint; b_layout::Cint; c_layout::Cint; d_layout::Cint
    c_type::Cint; d_type::Cint
    use_c::Cint
    addr_space::Cint
    alpha::Cfloat; beta::Cfloat
    lda::Int64; ldb::Int64; ldc::Int64; ldd::Int64
end

function mac!(d::DeviceBuffer{DT}, a::DeviceBuffer{Float16}, b::DeviceBuffer{Float16},
              c::Union{DeviceBuffer{CT},Nothing}; alpha=1f0, beta=1f0, a_layout=ColMajor, b_layout=ColMajor,
              c_layout=ColMajor, d_layout=ColMajor, addr_space=AS.Global) where {DT, CT}
    cty = c === nothing ? Float32 : CT
    desc = Ref(MacDesc(16, 16, 16, layout_code(a_layout), layout_code(b_layout), layout_code(c_layout),
                       layout_code(d_layout), dtype_code(cty), dtype_code(DT), c === nothing ? 0 : 1,
                       as_code(addr_space), alpha, beta, 16, 16, 16, 16))
    GC.@preserve a b c d check(ccall((:miw_wmma_mac, libmiwmma), Cint,
        (Ptr{MacDesc}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        desc, a.ptr, b.ptr, c === nothing ? C_NULL : c.ptr, d.ptr, current_stream()))
    return d
end

# ---- flatten / unflatten (src/device/cuda/wmma.jl:264-294): nested tuples of VecElements and
# scalars <-> one flat tuple.  Plain recursion on values; pinned by the exact equalities of
# test/device/wmma.jl:156-176.
flatten(x) = (x,)
flatten(x::VecElement) = (x.value,)
flatten(x::Tuple) = isempty(x) ? () : (flatten(first(x))..., flatten(Base.tail(x))...)

leaf_count(::Type{T}) where {T} = 1
leaf_count(::Type{T}) where {T <: Tuple} = sum(Int[leaf_count(F) for F in fieldtypes(T)])
rebuild(::Type{T}, x, at::Int) where {T} = convert(T, x[at])
rebuild(::Type{VecElement{T}}, x, at::Int) where {T} = VecElement{T}(x[at])
function rebuild(::Type{T}, x, at::Int) where {T <: Tuple}
    parts = Any[]
    for F in fieldtypes(T)
        push!(parts, rebuild(F, x, at))
        at += leaf_count(F)
    end
    return T(Tuple(parts))
end
unflatten(::Type{T}, x) where {T} = rebuild(T, x, 1)

# ---- the 52 low-level names of src/device/cuda/wmma.jl:104-257.  In the reference they wrap one
# NVVM intrinsic each and return the warp's registers as tuples; here each is one launch and the
# "registers" are the fragment image (a DeviceBuffer of 64 lanes x 4 elements).  Same names, same
# argument order: (src_addr, stride), (dst_addr, data, stride), (a, b, c).
const LL_LAYOUTS = (("col", ColMajor), ("row", RowMajor))
const LL_SPACES = (("", AS.Generic), ("shared", AS.Shared), ("global", AS.Global))
const LL_TYPES = (("f16", Float16), ("f32", Float32))
ll_name(parts...) = Symbol(join(filter(!isempty, collect(String, parts)), "_"))
low_level_names = Symbol[]

for (mat, U) in (("a", MatrixA), ("b", MatrixB), ("c", Accumulator)), (lname, L) in LL_LAYOUTS,
    (sname, A) in LL_SPACES, (tname, T) in LL_TYPES
    tname == "f32" && mat != "c" && continue          # Float32 only for C
    f = ll_name("llvm", "wmma", "load", mat, lname, "m16n16k16", sname, "stride", tname)
    @eval $f(src_addr::DevicePtr, stride) = load_image($U, $T, $L, $A, src_addr.addr, stride)
    @eval export $f
    push!(low_level_names, f)
end

for (lname, L) in LL_LAYOUTS, (sname, A) in LL_SPACES, (tname, T) in LL_TYPES
    f = ll_name("llvm", "wmma", "store", "d", lname, "m16n16k16", sname, "stride", tname)
    @eval $f(dst_addr::DevicePtr, data::DeviceBuffer, stride) = store_image($T, $L, $A, dst_addr.addr, data, stride)
    @eval export $f
    push!(low_level_names, f)
end

for (aname, LA) in LL_LAYOUTS, (bname, LB) in LL_LAYOUTS, (dname, DT) in LL_TYPES, (cname, CT) in LL_TYPES
    f = ll_name("llvm", "wmma", "mma", aname, bname, "m16n16k16", dname, cname)
    @eval $f(a::DeviceBuffer, b::DeviceBuffer, c::DeviceBuffer) = mma_image($LA, $LB, $CT, $DT, a, b, c)
    @eval export $f
    push!(low_level_names, f)
end
@assert length(low_level_names) == 52

llvm_wmma_load() = error("Cannot call llvm_wmma_load without values for placeholders!")
llvm_wmma_store() = error("Cannot call llvm_wmma_store without values for placeholders!")
llvm_wmma_mma() = error("Cannot call llvm_wmma_mma without values for placeholders!")
export llvm_wmma_load, llvm_wmma_store, llvm_wmma_mma

end # module WMMA

# ---------------------------------------------------------------------------- launch ------

struct KernelAttributes
    num_regs::Cint
    max_threads_per_block::Cint
    static_shared_bytes::Csize_t
    local_bytes::Csize_t
    const_bytes::Csize_t
end

"""
A kernel that can be launched: one compiled into libmiwmma.so (`hipfunction(name)`) or one of a code
object of your own (`kernel(CodeObject(path), name)`).  The HostKernel of src/execution.jl:205-219:
callable with the launch keywords `threads, blocks, shmem, stream, config`.
"""
struct HostKernel
    name::String
    fun::Ptr{Cvoid}
    owner::Any          # the CodeObject that must outlive the kernel, or nothing
end

"Names of the kernels compiled into the library."
function kernel_names()
    n = ccall((:miw_kernel_count, libmiwmma), Cint, ())
    buf = Vector{UInt8}(undef, 128)
    names = String[]
    for i in 0:n-1
        check(ccall((:miw_kernel_name, libmiwmma), Cint, (Cint, Ptr{UInt8}, Csize_t), i, buf, length(buf)))
        push!(names, unsafe_string(pointer(buf)))
    end
    return names
end

const kernel_cache = Dict{String,HostKernel}()
const kernel_cache_lock = ReentrantLock()

"cufunction (src/execution.jl:290-297): look a precompiled kernel up by name, cached."
function hipfunction(name::AbstractString)
    lock(kernel_cache_lock) do
        get!(kernel_cache, String(name)) do
            p = Ref{Ptr{Cvoid}}(C_NULL)
            check(ccall((:miw_kernel_lookup, libmiwmma), Cint, (Cstring, Ptr{Ptr{Cvoid}}), name, p))
            HostKernel(String(name), p[], nothing)
        end
    end
end

"A gfx950 code object compiled ahead of time (hipcc --genco): CuModule(image) of src/execution.jl:300-342."
mutable struct CodeObject
    handle::Ptr{Cvoid}
    function CodeObject(image::Vector{UInt8})
        p = Ref{Ptr{Cvoid}}(C_NULL)
        GC.@preserve image check(ccall((:miw_module_load, libmiwmma), Cint, (Ptr{Cvoid}, Csize_t, Ptr{Ptr{Cvoid}}),
                                       pointer(image), length(image), p))
        m = new(p[])
        finalizer(m) do x
            x.handle == C_NULL || ccall((:miw_module_unload, libmiwmma), Cint, (Ptr{Cvoid},), x.handle)
            x.handle = C_NULL
        end
        return m
    end
end
CodeObject(path::AbstractString) = CodeObject(read(path))

"CuFunction(mod, name)."
function kernel(m::CodeObject, name::AbstractString)
    p = Ref{Ptr{Cvoid}}(C_NULL)
    check(ccall((:miw_module_get_kernel, libmiwmma), Cint, (Ptr{Cvoid}, Cstring, Ptr{Ptr{Cvoid}}), m.handle, name, p))
    return HostKernel(String(name), p[], m)
end

function attributes(k::HostKernel)
    a = Ref{KernelAttributes}()
    check(ccall((:miw_kernel_attributes_get, libmiwmma), Cint, (Ptr{Cvoid}, Ptr{KernelAttributes}), k.fun, a))
    return a[]
end
"registers / memory / maxthreads of src/execution.jl:227-266."
registers(k::HostKernel) = Int(attributes(k).num_regs)
maxthreads(k::HostKernel) = Int(attributes(k).max_threads_per_block)
function memory(k::HostKernel)
    a = attributes(k)
    return (local=Int(a.local_bytes), shared=Int(a.static_shared_bytes), constant=Int(a.const_bytes))
end

"The occupancy API behind @cuda's config= callback (src/execution.jl:59-63): (blocks, threads)."
function launch_configuration(k::HostKernel; shmem::Integer=0)
    g, b = Ref{Cint}(0), Ref{Cint}(0)
    check(ccall((:miw_kernel_occupancy, libmiwmma), Cint, (Ptr{Cvoid}, Csize_t, Ptr{Cint}, Ptr{Cint}), k.fun, shmem, g, b))
    return (blocks=Int(g[]), threads=Int(b[]))
end

# cudaconvert (src/execution.jl:119-141): host object -> the value the kernel sees
hipconvert(a::DeviceBuffer) = a.ptr
hipconvert(p::DevicePtr) = Ptr{Cvoid}(p.addr)
hipconvert(x::Bool) = Cint(x)
hipconvert(x::Integer) = Clong(x)
hipconvert(x::Union{Int32,UInt32,Float16,Float32,Float64}) = x
hipconvert(x::AbstractFloat) = Float32(x)
hipconvert(x) = isbits(x) ? x : throw(ArgumentError("kernel argument of type $(typeof(x)) is not a bits value"))

dim3(x::Integer) = (Cuint(x), Cuint(1), Cuint(1))
dim3(x::Tuple) = (Cuint(x[1]), Cuint(length(x) > 1 ? x[2] : 1), Cuint(length(x) > 2 ? x[3] : 1))

function (k::HostKernel)(args...; threads=1, blocks=1, shmem::Integer=0, stream=C_NULL, config=nothing)
    if config !== nothing
        kw = config(k)
        threads = get(kw, :threads, threads)
        blocks = get(kw, :blocks, blocks)
        shmem = get(kw, :shmem, shmem)
    end
    boxes = Any[Ref(hipconvert(a)) for a in args]          # one slot per argument
    GC.@preserve args boxes begin
        slots = Ptr{Cvoid}[Base.unsafe_convert(Ptr{Cvoid}, b) for b in boxes]
        GC.@preserve slots check(ccall((:miw_launch, libmiwmma), Cint,
            (Ptr{Cvoid}, Ref{NTuple{3,Cuint}}, Ref{NTuple{3,Cuint}}, Cuint, Ptr{Cvoid}, Ptr{Ptr{Cvoid}}),
            k.fun, dim3(blocks), dim3(threads), shmem, stream_handle(stream),
            isempty(slots) ? Ptr{Ptr{Cvoid}}(C_NULL) : pointer(slots)))
    end
    return nothing
end

# A Julia function made of WMMA fragment operations "runs" as one wavefront: every operation inside
# is a launch on `stream`.  It has no launch-time LDS and no occupancy choice, so those keywords
# are refused instead of dropped.
function run_fragment_kernel(f, args...; threads=64, blocks=1, shmem::Integer=0, stream=C_NULL, config=nothing)
    config === nothing || throw(ArgumentError("config= needs a compiled kernel (hipfunction or a CodeObject kernel)"))
    shmem == 0 || throw(ArgumentError("shmem= needs a compiled kernel: a fragment function stages LDS tiles inside each operation"))
    (dim3(threads) == dim3(64) && dim3(blocks) == dim3(1)) ||
        throw(MIWError(Cint(-1), "a WMMA fragment kernel runs as one wavefront: threads=64, blocks=1"))
    with_stream(stream) do
        GC.@preserve args f(args...)
    end
end

launch(k::HostKernel, args...; kw...) = k(args...; kw...)
launch(name::AbstractString, args...; kw...) = hipfunction(name)(args...; kw...)
launch(f, args...; kw...) = run_fragment_kernel(f, args...; kw...)

"""
    @hip [threads=] [blocks=] [shmem=] [stream=] [config=] f(args...)

The `@cuda` of src/execution.jl:45-114.  `f` is a `HostKernel` (or the name of a kernel of the
library): launched with the given configuration, `config` being a callback `kernel -> (threads=,
blocks=, shmem=)`.  Or `f` is a Julia function written with the WMMA fragment operations: it runs
as one wavefront (threads must be 64, blocks 1) with every fragment operation inside launched on
`stream`, which is set for the running task only.
"""
macro hip(ex...)
    call = ex[end]
    Meta.isexpr(call, :call) || throw(ArgumentError("second argument to @hip should be a function call"))
    kws = Expr[]
    for kw in ex[1:end-1]
        Meta.isexpr(kw, :(=)) || throw(ArgumentError("expected keyword arguments before the call"))
        key, val = kw.args
        key in (:threads, :blocks, :shmem, :stream, :config) || throw(ArgumentError("Unsupported keyword argument '$key'"))
        push!(kws, Expr(:kw, key, esc(val)))
    end
    f, args = call.args[1], call.args[2:end]
    return :(launch($(esc(f)), $(map(esc, args)...); $(kws...)))
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

struct GemmVariantInfo
    name::NTuple{64,UInt8}
    block_m::Cint; block_n::Cint; block_k::Cint
    waves_m::Cint; waves_n::Cint
    stages::Cint
    lds_bytes::Cint
    fragment_ops::Cint
    f16_accumulate::Cint
    pingpong::Cint
end

struct GemmPart
    variant::Cint
    reserved::Cint
    m0::Int64; n0::Int64; k0::Int64
    m::Int64; n::Int64; k::Int64
end

function gemm_desc(M::Integer, N::Integer, K::Integer, ::Type{CT}, ::Type{DT}; alpha=1f0, beta=1f0,
                   a_layout=WMMA.ColMajor, b_layout=WMMA.ColMajor, c_layout=WMMA.ColMajor, d_layout=WMMA.ColMajor,
                   acc_type=Float32, acc_chunk=0, use_c=true, batch=1, variant=0, lda=0, ldb=0, ldc=0, ldd=0,
                   stride_a=0, stride_b=0, stride_c=0, stride_d=0) where {CT, DT}
    return GemmDesc(M, N, K, lda, ldb, ldc, ldd, WMMA.layout_code(a_layout), WMMA.layout_code(b_layout),
                    WMMA.layout_code(c_layout), WMMA.layout_code(d_layout), WMMA.dtype_code(CT), WMMA.dtype_code(DT),
                    WMMA.dtype_code(acc_type), acc_chunk, alpha, beta, use_c ? 1 : 0, batch,
                    stride_a, stride_b, stride_c, stride_d, variant)
end

"""
    gemm!(D, A, B, C, M, N, K; alpha=1, beta=1, a_layout=ColMajor, ..., acc_type=Float32, batch=1)

D = alpha*A*B + beta*C on the tiled MFMA kernels (asynchronous; call `synchronize()` before
reading D).  A, B are `DeviceBuffer{Float16}`; C, D `DeviceBuffer{Float16}` or `{Float32}`.
"""
function gemm!(D::DeviceBuffer{DT}, A::DeviceBuffer{Float16}, B::DeviceBuffer{Float16},
               C::Union{DeviceBuffer{CT},Nothing}, M::Integer, N::Integer, K::Integer;
               stream=C_NULL, kw...) where {DT, CT}
    desc = Ref(gemm_desc(M, N, K, C === nothing ? Float32 : CT, DT; use_c=C !== nothing, kw...))
    GC.@preserve A B C D check(ccall((:miw_gemm, libmiwmma), Cint,
        (Ptr{GemmDesc}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        desc, A.ptr, B.ptr, C === nothing ? C_NULL : C.ptr, D.ptr, stream_handle(stream)))
    return D
end

"Kernel variants of the library: id, name, tile, wavefronts, LDS slots and bytes, flags."
function gemm_variants()
    n = ccall((:miw_gemm_variant_count, libmiwmma), Cint, ())
    out = NamedTuple[]
    for v in 1:n
        info = Ref{GemmVariantInfo}()
        check(ccall((:miw_gemm_variant_info_get, libmiwmma), Cint, (Cint, Ptr{GemmVariantInfo}), v, info))
        i = info[]
        push!(out, (id=Int(v), name=cstring(i.name), block=(Int(i.block_m), Int(i.block_n), Int(i.block_k)),
                    waves=(Int(i.waves_m), Int(i.waves_n)), stages=Int(i.stages), lds_bytes=Int(i.lds_bytes),
                    fragment_ops=i.fragment_ops != 0, f16_accumulate=i.f16_accumulate != 0, pingpong=i.pingpong == 1, wave128=i.pingpong == 2))
    end
    return out
end

function pick_variant(desc::GemmDesc)
    v = Ref{Cint}(0)
    check(ccall((:miw_gemm_pick_variant, libmiwmma), Cint, (Ptr{GemmDesc}, Ptr{Cint}), Ref(desc), v))
    return Int(v[])
end

"The launches `gemm!` makes for this descriptor (one unless the sizes are ragged and cutting pays)."
function gemm_plan(desc::GemmDesc; in_place::Bool=false)
    parts = Vector{GemmPart}(undef, 64)
    n = Ref{Cint}(0)
    check(ccall((:miw_gemm_plan, libmiwmma), Cint, (Ptr{GemmDesc}, Cint, Ptr{GemmPart}, Cint, Ptr{Cint}),
                Ref(desc), in_place ? 1 : 0, parts, length(parts), n))
    return parts[1:min(Int(n[]), length(parts))]
end

function variant_supports(desc::GemmDesc, variant::Integer)
    ok = Ref{Cint}(0)
    check(ccall((:miw_gemm_variant_supports, libmiwmma), Cint, (Ptr{GemmDesc}, Cint, Ptr{Cint}), Ref(desc), variant, ok))
    return ok[] != 0
end

function acc_chunk(desc::GemmDesc)
    v = Ref{Cint}(0)
    check(ccall((:miw_gemm_acc_chunk, libmiwmma), Cint, (Ptr{GemmDesc}, Ptr{Cint}), Ref(desc), v))
    return Int(v[])
end

"(variant, acc_chunk) of the first launch gemm! makes for these operands (alignment and a C that is D count); no launch."
function gemm_resolve(desc::GemmDesc, A::DeviceBuffer, B::DeviceBuffer, C::Union{DeviceBuffer,Nothing}, D::DeviceBuffer)
    v, chunk = Ref{Cint}(0), Ref{Cint}(0)
    GC.@preserve A B C D check(ccall((:miw_gemm_resolve, libmiwmma), Cint,
        (Ptr{GemmDesc}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cint}, Ptr{Cint}),
        Ref(desc), A.ptr, B.ptr, C === nothing ? C_NULL : C.ptr, D.ptr, v, chunk))
    return Int(v[]), Int(chunk[])
end

"(slices, workspace bytes) of a split-K launch of this problem (splits = 0: chosen by the library)."
function splitk_workspace(desc::GemmDesc, splits::Integer=0)
    n, bytes = Ref{Cint}(0), Ref{Csize_t}(0)
    check(ccall((:miw_gemm_splitk_workspace, libmiwmma), Cint, (Ptr{GemmDesc}, Cint, Ptr{Cint}, Ptr{Csize_t}),
                Ref(desc), splits, n, bytes))
    return Int(n[]), Int(bytes[])
end

"Split-K GEMM through a caller workspace (`DeviceBuffer{Float32}` of at least splitk_workspace bytes)."
function gemm_splitk!(D::DeviceBuffer{DT}, A::DeviceBuffer{Float16}, B::DeviceBuffer{Float16},
                      C::Union{DeviceBuffer{CT},Nothing}, M::Integer, N::Integer, K::Integer,
                      workspace::DeviceBuffer{Float32}; splits::Integer=0, stream=C_NULL, kw...) where {DT, CT}
    desc = Ref(gemm_desc(M, N, K, C === nothing ? Float32 : CT, DT; use_c=C !== nothing, kw...))
    GC.@preserve A B C D workspace check(ccall((:miw_gemm_splitk, libmiwmma), Cint,
        (Ptr{GemmDesc}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Cint, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
        desc, A.ptr, B.ptr, C === nothing ? C_NULL : C.ptr, D.ptr, splits, workspace.ptr,
        length(workspace) * sizeof(Float32), stream_handle(stream)))
    return D
end

splitk_static_capacity() = Int(ccall((:miw_gemm_splitk_static_capacity, libmiwmma), Csize_t, ()))

"(slices, bytes of the static workspace) gemm_splitk_static! will use; touches no device."
function splitk_static_plan(desc::GemmDesc, splits::Integer=0)
    n, bytes = Ref{Cint}(0), Ref{Csize_t}(0)
    check(ccall((:miw_gemm_splitk_static_plan, libmiwmma), Cint, (Ptr{GemmDesc}, Cint, Ptr{Cint}, Ptr{Csize_t}),
                Ref(desc), splits, n, bytes))
    return Int(n[]), Int(bytes[])
end

"Split-K GEMM through the library's static device workspace: allocates nothing; calls that overlap on one GPU race."
function gemm_splitk_static!(D::DeviceBuffer{DT}, A::DeviceBuffer{Float16}, B::DeviceBuffer{Float16},
                             C::Union{DeviceBuffer{CT},Nothing}, M::Integer, N::Integer, K::Integer;
                             splits::Integer=0, stream=C_NULL, kw...) where {DT, CT}
    desc = Ref(gemm_desc(M, N, K, C === nothing ? Float32 : CT, DT; use_c=C !== nothing, kw...))
    GC.@preserve A B C D check(ccall((:miw_gemm_splitk_static, libmiwmma), Cint,
        (Ptr{GemmDesc}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Cint, Ptr{Cvoid}),
        desc, A.ptr, B.ptr, C === nothing ? C_NULL : C.ptr, D.ptr, splits, stream_handle(stream)))
    return D
end

"Per-launch durations in milliseconds (HIP events on the launch stream)."
function gemm_bench(D::DeviceBuffer, A::DeviceBuffer{Float16}, B::DeviceBuffer{Float16}, C::Union{DeviceBuffer,Nothing},
                    desc::GemmDesc; warmup::Integer=5, iters::Integer=20, stream=C_NULL)
    ms = Vector{Cfloat}(undef, iters)
    GC.@preserve A B C D ms check(ccall((:miw_gemm_bench, libmiwmma), Cint,
        (Ptr{GemmDesc}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Cint, Cint, Ptr{Cfloat}),
        Ref(desc), A.ptr, B.ptr, C === nothing ? C_NULL : C.ptr, D.ptr, stream_handle(stream), warmup, iters, ms))
    return ms
end

# ---------------------------------------------------------------------------- probes ------

"Matrix cores alone, register-resident operands (examples/peakflops.jl): TFLOP/s."
function mfma_peak_probe(iters::Integer=20000; stream=C_NULL)
    t = Ref{Cdouble}(0)
    check(ccall((:miw_mfma_peak_probe, libmiwmma), Cint, (Cint, Ptr{Cdouble}, Ptr{Cvoid}), iters, t, stream_handle(stream)))
    return t[]
end

"The same on operands that change every k-step: (TFLOP/s, shader MHz) under the power cap."
function mfma_power_probe(iters::Integer=20000; random_operands::Bool=true, stream=C_NULL)
    t, f = Ref{Cdouble}(0), Ref{Cdouble}(0)
    check(ccall((:miw_mfma_power_probe, libmiwmma), Cint, (Cint, Cint, Ptr{Cdouble}, Ptr{Cdouble}, Ptr{Cvoid}),
                iters, random_operands ? 1 : 0, t, f, stream_handle(stream)))
    return t[], f[]
end

"The in-library leg of test/perf/launch_overhead: (host µs, event µs) per iteration."
function launch_overhead_probe(iters::Integer=1000; threads::Integer=1000)
    cpu, gpu = Vector{Cfloat}(undef, iters), Vector{Cfloat}(undef, iters)
    check(ccall((:miw_launch_overhead_probe, libmiwmma), Cint, (Cint, Cint, Ptr{Cfloat}, Ptr{Cfloat}), iters, threads, cpu, gpu))
    return cpu, gpu
end

function copy_probe(dst::DeviceBuffer, src::DeviceBuffer, bytes::Integer; stream=C_NULL)
    check(ccall((:miw_copy_probe, libmiwmma), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}), dst.ptr, src.ptr, bytes, stream_handle(stream)))
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

and examples/wmma/low-level.jl:

function kernel_ll(a_dev, b_dev, c_dev, d_dev)
    a_frag = llvm_wmma_load_a_col_m16n16k16_global_stride_f16(pointer(a_dev), 16)
    b_frag = llvm_wmma_load_b_col_m16n16k16_global_stride_f16(pointer(b_dev), 16)
    c_frag = llvm_wmma_load_c_col_m16n16k16_global_stride_f32(pointer(c_dev), 16)
    d_frag = llvm_wmma_mma_col_col_m16n16k16_f32_f32(a_frag, b_frag, c_frag)
    llvm_wmma_store_d_col_m16n16k16_global_stride_f32(pointer(d_dev), d_frag, 16)
    return
end
@hip threads=64 kernel_ll(a_dev, b_dev, c_dev, d_dev)

A kernel of your own, written in HIP C++ with include/miwmma_fragment.hpp and built with
`hipcc --genco --offload-arch=gfx950` (cudanative.jl_amd/examples/user_kernel.hip):

mod = CodeObject(joinpath(@__DIR__, "..", "examples", "user_kernel.hsaco"))
k = kernel(mod, "user_mac")
@hip threads=64 blocks=1 k(a_dev, b_dev, c_dev, d_dev, 0.5f0)
=#
