# Replacement for the cuBLAS calls of src/knetarrays/linalg.jl.  NOT EXECUTED here.
#   linalg.jl:45,48  cublasSgemm_v2 / cublasDgemm_v2  -> gemm_32 / gemm_64 (hipBLASLt inside the library)
#   linalg.jl:63,66  cublasSaxpy_v2 / cublasDaxpy_v2  -> axpy_32 / axpy_64 (unit increments, the only use on this path)
#   linalg.jl:80,83  cublasSscal_v2 / cublasDscal_v2  -> scal_32 / scal_64
#   src/ops20_gpu/bmm.jl:46-50  cublasSgemmStridedBatched / cublasDgemmStridedBatched -> bmm_32 / bmm_64
# The shape logic of gemm! (size2, DimensionMismatch checks, lda/ldb/ldc) is kept verbatim from linalg.jl:26-43.

using .LibKnet8: libknet8, @knet8, knet8_stream

for (T, S) in ((Float32, 32), (Float64, 64))
    g = "gemm_$(S)_stream"
    @eval begin
        function _gemm!(transA::AbstractChar, transB::AbstractChar, m, n, k, alpha::$T, A::KnetArray{$T}, lda, B::KnetArray{$T}, ldb, beta::$T, C::KnetArray{$T}, ldc)
            rc = ccall(($g, libknet8), Cint,
                       (Cchar, Cchar, Cint, Cint, Cint, $T, Ptr{$T}, Cint, Ptr{$T}, Cint, $T, Ptr{$T}, Cint, Ptr{Cvoid}),
                       transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, knet8_stream())
            rc == 0 || error("libknet8 gemm failed")
            return C
        end
        # the last lines of bmm! (src/ops20_gpu/bmm.jl:40-52); everything above them in that function stays as it is
        function _bmm!(transA::AbstractChar, transB::AbstractChar, m, n, k, alpha::$T, A::KnetArray{$T}, lda, strideA, B::KnetArray{$T}, ldb, strideB,
                       beta::$T, C::KnetArray{$T}, ldc, strideC, bs)
            rc = ccall(($("bmm_$(S)_stream"), libknet8), Cint,
                       (Cchar, Cchar, Cint, Cint, Cint, $T, Ptr{$T}, Cint, Clonglong, Ptr{$T}, Cint, Clonglong, $T, Ptr{$T}, Cint, Clonglong, Cint, Ptr{Cvoid}),
                       transA, transB, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta, C, ldc, strideC, bs, knet8_stream())
            rc == 0 || error("libknet8 bmm failed")
            return C
        end
        function axpy!(n::Integer, alpha::Number, x::KnetArray{$T}, incx::Integer, y::KnetArray{$T}, incy::Integer)
            (incx == 1 && incy == 1) || error("libknet8 axpy supports unit increments only")
            length(x) == length(y) || throw(DimensionMismatch("$(map(size,(x,y)))"))
            @knet8($("axpy_$S"), (Cint, $T, Ptr{$T}, Ptr{$T}), n, $T(alpha), x, y)
            return y
        end
        function scal!(n::Integer, alpha::Number, x::KnetArray{$T}, incx::Integer)
            incx == 1 || error("libknet8 scal supports unit increment only")
            @knet8($("scal_$S"), (Cint, $T, Ptr{$T}), n, $T(alpha), x)
            return x
        end
    end
end
