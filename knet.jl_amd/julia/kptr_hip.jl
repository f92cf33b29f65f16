# Storage hooks for src/knetarrays/kptr.jl and src/knetarrays/copy.jl on the HIP build.  NOT EXECUTED here.
#
# kptr.jl:186-194  knetMalloc(nbytes)     -> knet8_malloc   (size-class pool over hipMalloc inside the library)
# kptr.jl:143-163  freeKnetPtr finalizer   -> knet8_free     (block goes back to the library's free list)
# kptr.jl:204-226  Knet.gc                 -> knet8_trim
# kptr.jl:254-255  meminfo                 -> knet8_meminfo
# copy.jl:6-11     copyto! H2D/D2H/D2D     -> knet8_memcpy(dst, src, nbytes, kind, stream)
# With these, KnetArray{T,N}(ptr::KnetPtr, dims) (karray.jl:53-56) is unchanged: `ptr.ptr` is a hipMalloc'd
# device pointer and `unsafe_convert(Ptr{T}, a)` (karray.jl:121-127) hands it to every @knet8 call as before.

using .LibKnet8: libknet8, knet8_stream

function knetMalloc(nbytes::Int)
    p = ccall((:knet8_malloc, libknet8), Ptr{Cvoid}, (Csize_t,), nbytes)
    p == C_NULL ? nothing : p
end

knetFree(p::Ptr{Cvoid}) = ccall((:knet8_free, libknet8), Cvoid, (Ptr{Cvoid},), p)

knetgc() = ccall((:knet8_trim, libknet8), Csize_t, ())

function knet8_meminfo()
    out = zeros(Csize_t, 4)  # bytes in use, bytes cached, hipMalloc calls, pool hits
    ccall((:knet8_meminfo, libknet8), Cvoid, (Ptr{Csize_t},), out)
    out
end

const H2D, D2H, D2D = Cint(1), Cint(2), Cint(3)
function knet8_memcpy!(dst, src, nbytes::Integer, kind::Cint)
    rc = ccall((:knet8_memcpy, libknet8), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Cint, Ptr{Cvoid}), dst, src, nbytes, kind, knet8_stream())
    rc == 0 || error("knet8_memcpy failed")
    dst
end
