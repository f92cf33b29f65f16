# Optional fused dense-layer primitive on top of the library's biasF_S / Fback_biasgrad_S entry points.  NOT EXECUTED here.
# The reference has no such op: a layer `relu.(w*x .+ b)` runs add_S_12, relu_S (and dropout_S) as separate launches
# (src/knetarrays/binary.jl:61-95, src/ops20_gpu/activation.jl:17-29, src/ops20_gpu/dropout.jl:12-21) and its gradient as
# dropback_S, reluback_S_11 and sum(dz;dims=2).  A model opts in by calling `biasact(relu, w*x, b)` instead of
# `relu.(w*x .+ b)`; everything else (KnetArray, @diff, the op tables) is untouched.

using .LibKnet8: @knet8
import AutoGrad: @primitive

for (T, S) in ((Float32, 32), (Float64, 64)), f in (:relu, :sigm, :tanh, :elu, :selu)
    fwd, bwd = "bias$(f)_$S", "$(f)back_biasgrad_$S"
    @eval begin
        function biasact(::typeof($f), z::KnetArray{$T,2}, b::KnetArray{$T})
            m, n = size(z); @assert length(b) == m
            y = similar(z)
            @knet8($fwd, (Cint, Cint, Ptr{$T}, Ptr{$T}, Ptr{$T}), m, n, z, b, y)
            return y
        end
        # returns (dz, db); the tape asks for the two gradients one after the other, so the pair is cached on dy
        function biasactback(::typeof($f), dy::KnetArray{$T,2}, y::KnetArray{$T,2}, b::KnetArray{$T})
            m, n = size(y)
            dz = similar(y); db = similar(b)
            @knet8($bwd, (Cint, Cint, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{$T}), m, n, dy, y, dz, db)
            return dz, db
        end
    end
end

const _biasact_cache = IdDict{Any,Any}()   # dy => (dz, db), emptied when the second gradient is taken
function _biasact_grads(f, dy, y, b)
    get!(() -> biasactback(f, dy, y, b), _biasact_cache, dy)
end
@primitive biasact(f, z, b),dy,y  nothing  _biasact_grads(f, dy, y, b)[1]  (g = _biasact_grads(f, dy, y, b)[2]; delete!(_biasact_cache, dy); g)

# relu + dropout in one pass each way: y holds U[0,1) on entry (rand!(y)), as for dropout! (src/ops20/dropout.jl:45-58).
for (T, S) in ((Float32, 32), (Float64, 64))
    @eval begin
        function biasreludrop!(p, z::KnetArray{$T,2}, b::KnetArray{$T}, y::KnetArray{$T,2})
            m, n = size(z)
            @knet8($("biasreludrop_$S"), (Cint, Cint, $T, Ptr{$T}, Ptr{$T}, Ptr{$T}), m, n, $T(p), z, b, y)
            return y
        end
        function dropreluback_biasgrad(p, dy::KnetArray{$T,2}, y::KnetArray{$T,2}, b::KnetArray{$T})
            m, n = size(y)
            dz = similar(y); db = similar(b)
            @knet8($("dropreluback_biasgrad_$S"), (Cint, Cint, $T, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{$T}), m, n, $T(p), dy, y, dz, db)
            return dz, db
        end
    end
end

# The whole layer in one call: y = f.(w*x .+ b) with f = relu or identity (gemm_bias_act_S folds bias and relu into the product's
# output stage for small products; large ones run hipBLASLt followed by one in-place pass).  `act`: 0 none, 1 relu.
for (T, S) in ((Float32, 32), (Float64, 64))
    @eval function dense!(y::KnetArray{$T,2}, w::KnetArray{$T,2}, x::KnetArray{$T,2}, b::KnetArray{$T}; act::Integer=1)
        m, k = size(w); n = size(x, 2)
        @assert size(x, 1) == k && size(y) == (m, n) && length(b) == m
        rc = ccall(($("gemm_bias_act_$(S)_stream"), LibKnet8.libknet8), Cint,
                   (UInt8, UInt8, Cint, Cint, Cint, $T, Ptr{$T}, Cint, Ptr{$T}, Cint, Ptr{$T}, Cint, Ptr{$T}, Cint, Ptr{Cvoid}),
                   'N', 'N', m, n, k, one($T), w, m, x, k, b, act, y, m, LibKnet8.knet8_stream())
        rc == 0 || LibKnet8.knet8_check()
        return y
    end
end

# The layer's whole backward pass in one call for small layers: dz = f'(y) .* dy on the fly, dw = dz*x', db = sum(dz;dims=2),
# dx = w'*dz (dense_back_S).  Returns false when the library declines (a layer too large for its small-matrix kernels): the caller
# then uses Fback_biasgrad_S and gemm! as before.
for (T, S) in ((Float32, 32), (Float64, 64))
    @eval function dense_back!(dw::KnetArray{$T,2}, db::KnetArray{$T}, dx::Union{KnetArray{$T,2},Nothing},
                               w::KnetArray{$T,2}, x::KnetArray{$T,2}, y::KnetArray{$T,2}, dy::KnetArray{$T,2}; act::Integer=1)
        m, k = size(w); n = size(x, 2)
        @assert size(x, 1) == k && size(y) == (m, n) && size(dy) == (m, n) && size(dw) == (m, k) && length(db) == m
        rc = ccall(($("dense_back_$(S)_stream"), LibKnet8.libknet8), Cint,
                   (Cint, Cint, Cint, Cint, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{Cvoid}),
                   act, m, n, k, w, x, y, dy, dw, db, dx === nothing ? C_NULL : dx, LibKnet8.knet8_stream())
        rc < 0 && LibKnet8.knet8_check()
        return rc == 0
    end
end

# Output layer of a classifier: from the scores z = w*x .+ b and Int32 labels (0 = skip), the mean loss (scale * sum of the losses,
# scale = 1/count), and with dz = scale*(softmax(z) - onehot): dw = dz*x', db = sum(dz;dims=2), dx = w'*dz -- one call
# (dense_nll_back_S) in place of nll -> logsoftmax -> getindex (src/ops20/loss.jl:37-41) and the layer's separate backward launches.
# Returns false when the library declines (more than 16 classes or a layer beyond its small-matrix kernels).
for (T, S) in ((Float32, 32), (Float64, 64))
    @eval function dense_nll_back!(mean::KnetArray{$T}, dw::KnetArray{$T,2}, db::KnetArray{$T}, dx::Union{KnetArray{$T,2},Nothing},
                                   w::KnetArray{$T,2}, x::KnetArray{$T,2}, z::KnetArray{$T,2}, labels::KnetArray{Int32}, scale::Real)
        m, k = size(w); n = size(x, 2)
        @assert size(x, 1) == k && size(z) == (m, n) && length(labels) == n && size(dw) == (m, k) && length(db) == m
        rc = ccall(($("dense_nll_back_$(S)_stream"), LibKnet8.libknet8), Cint,
                   (Cint, Cint, Cint, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{Cint}, $T, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{Cvoid}),
                   m, n, k, w, x, z, labels, $T(scale), dw, db, dx === nothing ? C_NULL : dx, C_NULL, mean, LibKnet8.knet8_stream())
        rc < 0 && LibKnet8.knet8_check()
        return rc == 0
    end
end

# The same with the output layer's forward product inside the launch (dense_head_S): scores z = w*x .+ b are formed in the kernel (and
# written to `z` when given).  At most 16 classes and 512 instances (Float64: 256); returns false when the library declines.
for (T, S) in ((Float32, 32), (Float64, 64))
    @eval function dense_head!(mean::KnetArray{$T}, dw::KnetArray{$T,2}, db::KnetArray{$T}, dx::Union{KnetArray{$T,2},Nothing},
                               w::KnetArray{$T,2}, b::KnetArray{$T}, x::KnetArray{$T,2}, labels::KnetArray{Int32}, scale::Real;
                               z::Union{KnetArray{$T,2},Nothing}=nothing)
        m, k = size(w); n = size(x, 2)
        @assert size(x, 1) == k && length(b) == m && length(labels) == n && size(dw) == (m, k) && length(db) == m
        rc = ccall(($("dense_head_$(S)_stream"), LibKnet8.libknet8), Cint,
                   (Cint, Cint, Cint, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{Cint}, $T, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{$T}, Ptr{Cvoid}),
                   m, n, k, w, b, x, labels, $T(scale), dw, db, dx === nothing ? C_NULL : dx, C_NULL, mean, z === nothing ? C_NULL : z,
                   LibKnet8.knet8_stream())
        rc < 0 && LibKnet8.knet8_check()
        return rc == 0
    end
end
