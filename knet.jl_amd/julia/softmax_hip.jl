# Replacement for the two cuDNN calls of src/ops20_gpu/softmax.jl:44-56.  NOT EXECUTED here.
# Everything else in that file (the dims logic `:10-42`, the @primitive1 lines `:58-59`, csb1/csb2) stays.
#
# cuDNN there runs MODE_INSTANCE on TD4(x) = (1,1,m,n): softmax down each contiguous column of an m x n
# column-major matrix; algo LOG -> logsoftmax_S / logsoftmaxback_S, ACCURATE (and FAST) -> softmax_S / softmaxback_S.

using .LibKnet8: @knet8

for (T, S) in ((Float32, 32), (Float64, 64))
    fwd_log, fwd_acc = "logsoftmax_$S", "softmax_$S"
    bwd_log, bwd_acc = "logsoftmaxback_$S", "softmaxback_$S"
    @eval begin
        function _cudnnSoftmaxForward(x::KnetArray{$T}; algo)
            n = size(x, ndims(x)); m = div(length(x), n)          # TD4: (1,1,m,n)
            y = similar(x)
            if algo == CUDNN_SOFTMAX_LOG
                @knet8($fwd_log, (Cint, Cint, Ptr{$T}, Ptr{$T}), m, n, x, y)
            else
                @knet8($fwd_acc, (Cint, Cint, Ptr{$T}, Ptr{$T}), m, n, x, y)
            end
            return y
        end
        function _cudnnSoftmaxBackward(y::KnetArray{$T}, dy::KnetArray{$T}; algo)
            n = size(y, ndims(y)); m = div(length(y), n)
            dx = similar(y)
            if algo == CUDNN_SOFTMAX_LOG
                @knet8($bwd_log, (Cint, Cint, Ptr{$T}, Ptr{$T}, Ptr{$T}), m, n, y, dy, dx)
            else
                @knet8($bwd_acc, (Cint, Cint, Ptr{$T}, Ptr{$T}, Ptr{$T}), m, n, y, dy, dx)
            end
            return dx
        end
        # Optional: nll and its gradient in one pass over the scores (no libknet8 counterpart in the reference).
        # labels::KnetArray{Int32} holds 1-based classes, 0 = skip; returns (dx, per-instance losses).
        function nll_logsoftmax_back(scores::KnetArray{$T,2}, labels::KnetArray{Int32}, scale::$T)
            m, n = size(scores)
            dx = similar(scores); loss = similar(scores, (n,))
            @knet8($("nll_logsoftmax_back_$S"), (Cint, Cint, Ptr{$T}, Ptr{Int32}, $T, Ptr{$T}, Ptr{$T}), m, n, scores, labels, scale, dx, loss)
            return dx, loss
        end
    end
end
