# Replacement for src/libknet8/LibKnet8.jl of Knet.jl when libknet8.so is the MI355X (gfx950) build.
# NOT EXECUTED in this repository's environment (no Julia toolchain there): reviewed source only.
#
# What changes relative to the reference file: the library is located the same way (`:7`), but the
# stream appended to every call is a HIP stream handle (Ptr{Cvoid}) instead of CUDA.stream(), and the
# macros no longer go through CUDA.jl.  Everything that calls `@knet8` / `@knet8r` stays as it is.
module LibKnet8

export libknet8, @knet8, @knet8r, knet8_stream, knet8_check

using Libdl

const libknet8 = Libdl.find_library(["libknet8"], [get(ENV, "KNET8_LIBDIR", joinpath(@__DIR__, "..", "lib"))])

include("ops.jl")  # the reference's operator tables (unary_ops, binary_ops, reduction_ops ...) are used unchanged by the dispatch loops

# Task-local HIP stream handle; C_NULL is the null stream.  (The reference uses CUDA.stream().)
knet8_stream() = get(task_local_storage(), :knet8_stream, C_NULL)::Ptr{Cvoid}

macro knet8(fun, argtypes, argvalues...)
    f = string(fun, "_stream")
    at = Expr(:tuple, argtypes.args..., :(Ptr{Cvoid}))
    quote
        ccall(($f, libknet8), Nothing, $(esc(at)), $(map(esc, argvalues)...), knet8_stream())
    end
end

macro knet8r(fun, returntype, argtypes, argvalues...)  # `_20` reductions return T by value and block
    f = string(fun, "_stream")
    at = Expr(:tuple, argtypes.args..., :(Ptr{Cvoid}))
    quote
        ccall(($f, libknet8), $(esc(returntype)), $(esc(at)), $(map(esc, argvalues)...), knet8_stream())
    end
end

# The reference leaves libknet8 calls unchecked (errmsg=false, `:54`).  This build records failures; call this
# after a batch of launches to turn a recorded failure into a Julia error.
function knet8_check()
    p = ccall((:knet8_last_error, libknet8), Cstring, ())
    p == C_NULL || error("libknet8: ", unsafe_string(p))
end

end # module
