# permutedims!/permutedims for KnetArray on the HIP build: replaces the CuArray detour of src/knetarrays/reshape.jl:18 and the
# cuDNN/cuBLAS transposes of src/knetarrays/linalg.jl:95-113.  NOT EXECUTED here.
#
# reshape.jl:18   permutedims!(y::KnetArray, x::KnetArray, perm) = (permutedims!(CuArray(y), CuArray(x), perm); y)  -> permutedims_S
# linalg.jl:96    _transpose(x::KnetMatrix) = _transpose!(similar(x,(size(x,2),size(x,1))),x)                        -> transpose_S
# `dims` and `perm` are host Int32 vectors read during the call (1-based perm, as Julia passes it); up to 8 dimensions.

import Base: permutedims!
using .LibKnet8: @knet8

for (T, S) in ((Float32, 32), (Float64, 64))
    @eval begin
        function permutedims!(y::KnetArray{$T}, x::KnetArray{$T}, perm)
            nd = ndims(x)
            (nd == length(perm) && isperm(perm)) || throw(ArgumentError("no valid permutation of dimensions"))
            nd <= 8 || throw(ArgumentError("permutedims! of KnetArray supports at most 8 dimensions"))
            size(y) == ntuple(i -> size(x, perm[i]), nd) || throw(DimensionMismatch("destination tensor of incorrect size"))
            dims = Int32[size(x)...]
            p = Int32[perm...]
            GC.@preserve dims p begin
                @knet8($("permutedims_$S"), (Cint, Ptr{Cint}, Ptr{Cint}, Ptr{$T}, Ptr{$T}), nd, pointer(dims), pointer(p), x, y)
            end
            return y
        end
        function _transpose!(y::KnetMatrix{$T}, x::KnetMatrix{$T})
            @knet8($("transpose_$S"), (Cint, Cint, Ptr{$T}, Ptr{$T}), size(x, 1), size(x, 2), x, y)
            return y
        end
    end
end
