# rand!/randn!/seed! for KnetArray on the HIP build: replaces the CuArray detour of src/knetarrays/random.jl:5-18.
# NOT EXECUTED here.
#
# random.jl:5   rand!(a::KnetArray)=(rand!(CuArray(a)); a)     -> rand_32 / rand_64   (U[0,1), Philox4x32-10 inside the library)
# random.jl:6   randn!(a::KnetArray)=(randn!(CuArray(a)); a)   -> randn_32 / randn_64
# random.jl:14  seed!(x): CUDA.seed!(x)                        -> knet8_seed(x)
# src/ops20_gpu/dropout.jl:13-14 (`CUDA.seed!(seed); rand!(y)`) then works unchanged on top of these.

import Random: rand!, randn!, Random
using .LibKnet8: libknet8, @knet8

for (T, S) in ((Float32, 32), (Float64, 64))
    @eval begin
        rand!(a::KnetArray{$T})  = (@knet8($("rand_$S"),  (Cint, Ptr{$T}), length(a), a); a)
        randn!(a::KnetArray{$T}) = (@knet8($("randn_$S"), (Cint, Ptr{$T}), length(a), a); a)
        # explicit stream position, for reproducible masks and for code captured into a hipGraph
        rand!(a::KnetArray{$T}, seed::Integer, offset::Integer) =
            (@knet8($("rand_seeded_$S"), (Cint, Culonglong, Culonglong, Ptr{$T}), length(a), seed % UInt64, offset % UInt64, a); a)
    end
end

"Seed the device stream (if a GPU is in use) and Julia's own generator, as Knet.seed! does."
function seed!(x)
    ccall((:knet8_seed, libknet8), Cvoid, (Culonglong,), x % UInt64)
    Random.seed!(x)
end
