#!/usr/bin/env python3
"""Generator of libknet8's gfx950 HIP sources and of its public header.

Plays the role of the reference's src/libknet8/build.jl:42-82 + ops.jl: the operator tables below
are the configuration; each row becomes a device functor plus the ``extern "C"`` entry points
(``NAME_stream(..., hipStream_t)`` and the plain ``NAME`` twin) that Knet's ``@knet8`` ccall layer
binds (src/libknet8/LibKnet8.jl:50-62).  The kernels themselves are the hand-written templates in
knet8_elementwise.h / knet8_reduce.h / knet8_softmax.h / knet8_index.h.

Expressions follow the reference's CPU ``Array`` path (src/ops20/activation.jl, src/ops21/activation.jl)
where it differs from the expressions compiled into the reference's CUDA kernels
(src/libknet8/ops.jl): ``>=`` branch tests for elu/selu, selu constants rounded to T before use,
NaN-propagating relu, division (not multiplication by a reciprocal) in dropout.

Usage:  python gen_knet8.py   (writes gen/*.hip next to this file and include/knet8.h at the repo root)
"""
import os

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
GEN = os.path.join(HERE, "gen")
HEADER = os.path.join(ROOT, "include", "knet8.h")

TYPES = [("float", "32"), ("double", "64")]

LAMBDA01 = "1.0507009873554805"
LAMBDAALPHA01 = "1.7580993408473773"
SQRT2 = "1.4142135623730951"
SQRT2PI = "2.5066282746310002"

# name, body (statements ending in a return; `xi` is the input), reference citation
UNARY_OPS = [
    ("relu", "return xi != xi ? xi : (xi > T(0) ? xi : T(0));", "src/ops20/activation.jl:26, src/libknet8/ops.jl:76"),
    ("sigm", "if (xi >= T(0)) return T(1) / (T(1) + kexp(-xi)); const T z = kexp(xi); return z / (T(1) + z);",
     "src/ops20/activation.jl:55, src/libknet8/ops.jl:78"),
    ("tanh", "return ktanh(xi);", "src/libknet8/ops.jl:61"),
    ("tanh_", "return ktanh(xi);", "src/ops21/activation.jl:186, src/libknet8/ops.jl:62"),
    ("elu", "return xi >= T(0) ? xi : kexp(xi) - T(1);", "src/ops20/activation.jl:12, src/libknet8/ops.jl:72"),
    ("selu", "return xi >= T(0) ? T(%s) * xi : T(%s) * (kexp(xi) - T(1));" % (LAMBDA01, LAMBDAALPHA01),
     "src/ops20/activation.jl:39, src/libknet8/ops.jl:77"),
    ("gelu", "const T a = xi / T(%s); const T b = T(1) + kerf(a); const T c = xi * b; return c / T(2);" % SQRT2,
     "src/ops21/activation.jl:37, src/libknet8/ops.jl:73"),
    ("hardsigmoid", "return xi <= T(-3) ? T(0) : xi >= T(3) ? T(1) : (xi + T(3)) / T(6);",
     "src/ops21/activation.jl:61, src/libknet8/ops.jl:74"),
    ("hardswish", "if (xi <= T(-3)) return T(0); if (xi >= T(3)) return xi; const T a = xi + T(3); const T b = xi * a; return b / T(6);",
     "src/ops21/activation.jl:81, src/libknet8/ops.jl:75"),
    ("swish", "T s; if (xi >= T(0)) s = T(1) / (T(1) + kexp(-xi)); else { const T z = kexp(xi); s = z / (T(1) + z); } return xi * s;",
     "src/ops21/activation.jl:170, src/libknet8/ops.jl:79"),
    ("exp", "return kexp(xi);", "src/libknet8/ops.jl:26"),
    ("log", "return klog(xi);", "src/libknet8/ops.jl:40"),
    ("sqrt", "return ksqrt(xi);", "src/libknet8/ops.jl:58"),
    ("neg", "return -xi;", "src/libknet8/ops.jl:49"),
    ("abs", "return xi < T(0) ? -xi : xi;", "src/libknet8/ops.jl:8"),
    ("abs2", "return xi * xi;", "src/libknet8/ops.jl:7"),
    ("sign", "return xi > T(0) ? T(1) : xi < T(0) ? T(-1) : T(0);", "src/libknet8/ops.jl:55"),
    ("invx", "return T(1) / xi;", "src/libknet8/ops.jl:71"),
    ("one", "return T(1);", "src/libknet8/ops.jl:52"),
    ("copy", "return xi;", "the contiguous case of xcopy, src/libknet8/cuda1.jl:130-165 (also the known-size 1R+1W kernel used to calibrate HBM counters)"),
    ("zero", "return T(0);", "src/libknet8/ops.jl:67"),
    # the plain libm rows of the same table (src/libknet8/ops.jl:6-66)
    ("acos", "return kacos(xi);", "src/libknet8/ops.jl:6-66 (acos)"),
    ("acosh", "return kacosh(xi);", "src/libknet8/ops.jl:6-66 (acosh)"),
    ("asin", "return kasin(xi);", "src/libknet8/ops.jl:6-66 (asin)"),
    ("asinh", "return kasinh(xi);", "src/libknet8/ops.jl:6-66 (asinh)"),
    ("atan", "return katan(xi);", "src/libknet8/ops.jl:6-66 (atan)"),
    ("atanh", "return katanh(xi);", "src/libknet8/ops.jl:6-66 (atanh)"),
    ("cbrt", "return kcbrt(xi);", "src/libknet8/ops.jl:6-66 (cbrt)"),
    ("ceil", "return kceil(xi);", "src/libknet8/ops.jl:6-66 (ceil)"),
    ("cos", "return kcos(xi);", "src/libknet8/ops.jl:6-66 (cos)"),
    ("cosh", "return kcosh(xi);", "src/libknet8/ops.jl:6-66 (cosh)"),
    ("cospi", "return kcospi(xi);", "src/libknet8/ops.jl:6-66 (cospi)"),
    ("erf", "return kerf(xi);", "src/libknet8/ops.jl:6-66 (erf)"),
    ("erfc", "return kerfc(xi);", "src/libknet8/ops.jl:6-66 (erfc)"),
    ("erfcinv", "return kerfcinv(xi);", "src/libknet8/ops.jl:6-66 (erfcinv)"),
    ("erfcx", "return kerfcx(xi);", "src/libknet8/ops.jl:6-66 (erfcx)"),
    ("erfinv", "return kerfinv(xi);", "src/libknet8/ops.jl:6-66 (erfinv)"),
    ("exp10", "return kexp10(xi);", "src/libknet8/ops.jl:6-66 (exp10)"),
    ("exp2", "return kexp2(xi);", "src/libknet8/ops.jl:6-66 (exp2)"),
    ("expm1", "return kexpm1(xi);", "src/libknet8/ops.jl:6-66 (expm1)"),
    ("floor", "return kfloor(xi);", "src/libknet8/ops.jl:6-66 (floor)"),
    ("log10", "return klog10(xi);", "src/libknet8/ops.jl:6-66 (log10)"),
    ("log1p", "return klog1p(xi);", "src/libknet8/ops.jl:6-66 (log1p)"),
    ("log2", "return klog2(xi);", "src/libknet8/ops.jl:6-66 (log2)"),
    ("sin", "return ksin(xi);", "src/libknet8/ops.jl:6-66 (sin)"),
    ("sinh", "return ksinh(xi);", "src/libknet8/ops.jl:6-66 (sinh)"),
    ("sinpi", "return ksinpi(xi);", "src/libknet8/ops.jl:6-66 (sinpi)"),
    ("tan", "return ktan(xi);", "src/libknet8/ops.jl:6-66 (tan)"),
    ("trunc", "return ktrunc(xi);", "src/libknet8/ops.jl:6-66 (trunc)"),
    ("round", "return krint(xi);", "src/libknet8/ops.jl:52; ties go to the even neighbour as Julia's round does on the CPU path (the CUDA kernel rounds them away from zero)"),
    ("j0", "return kj0(xi);", "src/libknet8/ops.jl:31 (j0)"),
    ("j1", "return kj1(xi);", "src/libknet8/ops.jl:32 (j1)"),
    ("y0", "return ky0(xi);", "src/libknet8/ops.jl:63 (y0)"),
    ("y1", "return ky1(xi);", "src/libknet8/ops.jl:64 (y1)"),
    ("lgamma", "return klgamma(xi);", "src/libknet8/ops.jl:34"),
    ("gamma_impl", "return ktgamma(xi);", "src/libknet8/ops.jl:33 (gamma_impl, src/libknet8/gamma.jl)"),
    ("digamma_impl", "return kdigamma<T>(xi);", "src/libknet8/ops.jl:35, src/libknet8/gamma.jl:72-124 (poles return the largest finite T)"),
    ("trigamma_impl", "return ktrigamma<T>(xi);", "src/libknet8/ops.jl:36, src/libknet8/gamma.jl:221-239 (zeta(2,x); poles return the largest finite T)"),
]

# Unary ops with an integer degree NAME_S(n, d, x, y): name, device routine, citation (src/libknet8/ops.jl:138-141).
INT_DEGREE_OPS = [
    ("jn", "kbesselj", "src/libknet8/ops.jl:139, src/libknet8/cuda1.jl:49-79 (besselj(d,x), any integer d)"),
    ("yn", "kbessely", "src/libknet8/ops.jl:140, src/libknet8/cuda1.jl:49-79 (bessely(d,x); NaN for x < 0)"),
]

# name, body in terms of (xi, yi), citation.  Used for the _01, _11 and _12/_13 entry points.
BINARY_OPS = [
    ("add", "return xi + yi;", "src/libknet8/ops.jl:88"),
    ("sub", "return xi - yi;", "src/libknet8/ops.jl:89"),
    ("mul", "return xi * yi;", "src/libknet8/ops.jl:90"),
    ("div", "return xi / yi;", "src/libknet8/ops.jl:91"),
    ("max", "return xi > yi ? xi : yi;", "src/libknet8/ops.jl:93"),
    ("min", "return xi < yi ? xi : yi;", "src/libknet8/ops.jl:94"),
    ("pow", "return kpow(xi, yi);", "src/libknet8/ops.jl:92"),
    ("eq", "return xi == yi ? T(1) : T(0);", "src/libknet8/ops.jl:95"),
    ("ne", "return xi != yi ? T(1) : T(0);", "src/libknet8/ops.jl:96"),
    ("gt", "return xi > yi ? T(1) : T(0);", "src/libknet8/ops.jl:97"),
    ("ge", "return xi >= yi ? T(1) : T(0);", "src/libknet8/ops.jl:98"),
    ("lt", "return xi < yi ? T(1) : T(0);", "src/libknet8/ops.jl:99"),
    ("le", "return xi <= yi ? T(1) : T(0);", "src/libknet8/ops.jl:100"),
]

FUSED_ACTS = ["relu", "sigm", "tanh", "elu", "selu"]

# Two-input gradients NAME_S_11(n, dy, y, dx): xi = dy, yi = y.
BACK11_OPS = [
    ("invxback", "const T a = -xi; const T b = a * yi; return b * yi;", "src/libknet8/ops.jl:115 (-dy*y*y, the gradient of the deprecated invx, src/ops20/activation.jl:60-63)"),
    ("reluback", "return yi > T(0) ? xi : T(0);", "src/ops20/activation.jl:27, src/libknet8/ops.jl:118"),
    ("sigmback", "const T a = xi * yi; const T b = T(1) - yi; return a * b;", "src/ops20/activation.jl:56, src/libknet8/ops.jl:120"),
    ("tanhback", "const T a = yi * yi; const T b = T(1) - a; return xi * b;", "src/ops20_gpu/activation.jl:11, src/libknet8/ops.jl:121"),
    ("eluback", "if (yi >= T(0)) return xi; const T b = T(1) + yi; return xi * b;", "src/ops20/activation.jl:13, src/libknet8/ops.jl:116"),
    ("seluback", "if (yi >= T(0)) return xi * T(%s); const T b = yi + T(%s); return xi * b;" % (LAMBDA01, LAMBDAALPHA01),
     "src/ops20/activation.jl:40, src/libknet8/ops.jl:119"),
]

# The reference's binary table also carries geluback and swishback with xi = x, yi = dy (src/libknet8/ops.jl:110,116): same
# arithmetic as the three-input forms below.
def _back_as_binary(name):
    body = [b for n, b, _ in BACK111_OPS if n == name][0]
    return "const T x = xi; const T dy = yi; " + body


# Three-input gradients NAME_S_111(n, x, y, dy, dx).
BACK111_OPS = [
    ("eluback", "if (y >= T(0)) return dy; const T b = T(1) + y; return dy * b;", "src/ops21/activation.jl:17, src/libknet8/ops.jl:126"),
    ("seluback", "if (y >= T(0)) return dy * T(%s); const T b = y + T(%s); return dy * b;" % (LAMBDA01, LAMBDAALPHA01),
     "src/ops21/activation.jl:130, src/libknet8/ops.jl:132"),
    ("sigmback", "const T a = dy * y; const T b = T(1) - y; return a * b;", "src/ops21/activation.jl:152, src/libknet8/ops.jl:133"),
    ("tanh_back", "const T a = y * y; const T b = T(1) - a; return dy * b;", "src/ops21/activation.jl:187, src/libknet8/ops.jl:134"),
    ("geluback", "const T a = x / T(%s); const T b = (T(1) + kerf(a)) / T(2); const T x2 = x * x; const T e = kexp(-x2 / T(2)); "
                 "const T c = (x * e) / T(%s); const T d = b + c; return dy * d;" % (SQRT2, SQRT2PI),
     "src/ops21/activation.jl:38, src/libknet8/ops.jl:127"),
    ("hardsigmoidback", "const T g = x <= T(-3) ? T(0) : x >= T(3) ? T(0) : T(1.0 / 6.0); return dy * g;",
     "src/ops21/activation.jl:62, src/libknet8/ops.jl:128"),
    ("hardswishback", "T g; if (x <= T(-3)) g = T(0); else if (x >= T(3)) g = T(1); else { const T a = T(2) * x; const T b = a + T(3); g = b / T(6); } return dy * g;",
     "src/ops21/activation.jl:82, src/libknet8/ops.jl:129"),
    ("swishback", "T g; if (x >= T(0)) { const T z = kexp(-x); const T zx = z * x; const T num = (zx + z) + T(1); const T d = z + T(1); g = num / (d * d); } "
                  "else { const T z = kexp(x); const T s = (x + z) + T(1); const T num = z * s; const T d = z + T(1); g = num / (d * d); } return dy * g;",
     "src/ops21/activation.jl:171, src/libknet8/ops.jl:135"),
]

BACKBIN_OPS = [("geluback", _back_as_binary("geluback"), "src/libknet8/ops.jl:110 (xi = x, yi = dy)"),
               ("swishback", _back_as_binary("swishback"), "src/libknet8/ops.jl:116 (xi = x, yi = dy)")]

# Every row of the reference's binary table: the generators of the scalar and broadcast forms loop over all of them
# (src/libknet8/cuda01.jl:32, cuda12.jl:40, cuda13.jl:190, cuda16.jl:105, cuda17.jl:70), the gradient rows included.
ALL_BINARY_OPS = BINARY_OPS + BACK11_OPS + BACKBIN_OPS

# Fused optimizer updates: name, scalar parameters (all of type T, derived on the host exactly as the Julia code derives
# them: T(-lr), T(1-rho), T(1-beta1^t) ...), arrays (in order), write mask, body on v[...], citation.  Each body is the
# per-element sequence of the reference's lmul!/axpy!/broadcast chain, one rounding per operation.
OPTIMIZER_OPS = [
    ("momentum", ["nlr", "gamma"], ["g", "vel", "w"], 0b110,
     "const T v1 = gamma * v[1]; const T p = nlr * v[0]; const T v2 = v1 + p; v[1] = v2; v[2] = v[2] + v2;",
     "src/train20/update.jl:517-522"),
    ("nesterov", ["nlr", "gamma", "opg"], ["g", "vel", "w"], 0b110,
     "const T v1 = gamma * v[1]; const T m1 = T(-1) * v1; const T w1 = v[2] + m1; const T p = nlr * v[0]; const T v2 = v1 + p; "
     "const T q = opg * v2; v[1] = v2; v[2] = w1 + q;",
     "src/train20/update.jl:525-531"),
    ("adagrad", ["nlr", "eps"], ["g", "G", "w"], 0b110,
     "const T gg = v[0] * v[0]; const T G1 = v[1] + gg; const T t = G1 + eps; const T q = v[0] / ksqrt(t); const T p = nlr * q; v[1] = G1; v[2] = v[2] + p;",
     "src/train20/update.jl:533-538"),
    ("rmsprop", ["nlr", "rho", "omr", "eps"], ["g", "G", "w"], 0b110,
     "const T G1 = rho * v[1]; const T gg = v[0] * v[0]; const T a = omr * gg; const T G2 = G1 + a; const T t = G2 + eps; const T q = v[0] / ksqrt(t); "
     "const T p = nlr * q; v[1] = G2; v[2] = v[2] + p;",
     "src/train20/update.jl:540-546"),
    ("adadelta", ["nlr", "rho", "omr", "eps"], ["g", "G", "delta", "w"], 0b1110,
     "const T G1 = rho * v[1]; const T gg = v[0] * v[0]; const T a = omr * gg; const T G2 = G1 + a; const T sd = ksqrt(v[2] + eps); const T num = v[0] * sd; "
     "const T dw = num / ksqrt(G2 + eps); const T d1 = rho * v[2]; const T dd = dw * dw; const T b = omr * dd; const T p = nlr * dw; "
     "v[1] = G2; v[2] = d1 + b; v[3] = v[3] + p;",
     "src/train20/update.jl:548-557"),
    ("adam", ["nlr", "beta1", "omb1", "beta2", "omb2", "c1", "c2", "eps"], ["g", "fstm", "scndm", "w"], 0b1110,
     "const T m1 = beta1 * v[1]; const T a = omb1 * v[0]; const T m2 = m1 + a; const T s1 = beta2 * v[2]; const T gg = v[0] * v[0]; const T b = omb2 * gg; "
     "const T s2 = s1 + b; const T mc = m2 / c1; const T sc = s2 / c2; const T den = ksqrt(sc) + eps; const T q = mc / den; const T p = nlr * q; "
     "v[1] = m2; v[2] = s2; v[3] = v[3] + p;",
     "src/train20/update.jl:559-570"),
]

# Reduction operators: order and meaning of src/libknet8/ops.jl:144-156.
REDUCTION_OPS = [("sum", "RedSum"), ("prod", "RedProd"), ("maximum", "RedMaximum"), ("minimum", "RedMinimum"),
                 ("sumabs", "RedSumabs"), ("sumabs2", "RedSumabs2"), ("maxabs", "RedMaxabs"), ("minabs", "RedMinabs"),
                 ("countnz", "RedCountnz")]

BANNER = "// GENERATED by knet.jl_amd/csrc/gen_knet8.py -- edit the tables there, not this file.\n"


class Out:
    """Collects the HIP source of one translation unit and the matching header declarations."""

    def __init__(self):
        self.src = []
        self.decl = []

    def entry(self, name, ret, params, call, cite, guard="", body=None):
        """Emit NAME_stream(params..., hipStream_t) and the plain NAME twin (null stream)."""
        plist = ", ".join("%s %s" % (t, n) for t, n in params)
        pnames = ", ".join(n for _, n in params)
        sep = ", " if params else ""
        self.decl.append("/* replaces %s */" % cite)
        self.decl.append("KNET8_API %s %s_stream(%s%shipStream_t stream);" % (ret, name, plist, sep))
        self.decl.append("KNET8_API %s %s(%s);" % (ret, name, plist))
        if body is None:
            body = "  %s%s;\n  knet8::check_launch(\"%s\");" % (guard, call, name)
        self.src.append("extern \"C\" KNET8_API %s %s_stream(%s%shipStream_t stream) {\n%s\n}" % (ret, name, plist, sep, body))
        r = "return " if ret != "void" else ""
        self.src.append("extern \"C\" KNET8_API %s %s(%s) { %s%s_stream(%s%s0); }\n" % (ret, name, plist, r, name, pnames, sep))


PRELUDE = BANNER + """#include "../knet8_runtime.h"
#include "../knet8_elementwise.h"
#include "../knet8_special.h"
#include "../knet8_random.h"
#include "../knet8_broadcast.h"
#include "../knet8_reduce.h"
#include "../knet8_fused.h"
#include "../knet8_dense.h"
#include "../knet8_softmax.h"
#include "../knet8_index.h"
#include "../knet8_transpose.h"
#include "../knet8_permute.h"
using namespace knet8;

"""


def functor(name, args, body, extra_fields=""):
    return ("template <typename T> struct %s {\n%s  __device__ __forceinline__ T operator()(%s) const { %s }\n};\n"
            % (name, extra_fields, ", ".join("T " + a for a in args), body))


def binary_functors():
    out = []
    for name, body, cite in BINARY_OPS + BACKBIN_OPS:
        out.append(functor("Op2_" + name, ["xi", "yi"], body))
    for name, body, cite in BACK11_OPS:
        out.append(functor("Op11_" + name, ["xi", "yi"], body))
        out.append("template <typename T> using Op2_%s = Op11_%s<T>;\n" % (name, name))
    return "\n".join(out)


def gen_broadcast():
    o = Out()
    s = o.src
    s.append(PRELUDE)
    s.append(binary_functors())
    o.decl.append("\n/* ---- vector broadcast: operand k is full size or a vector along one dim, read as v[(i/s)%n]\n"
                  "   -- src/libknet8/cuda12.jl:18-34; the _13 forms (src/libknet8/cuda13.jl:44-184) take the full array first ---- */")
    for name, body, cite in ALL_BINARY_OPS:
        s.append("template <typename T> struct Op2r_%s { __device__ __forceinline__ T operator()(T full, T vec) const { return Op2_%s<T>()(vec, full); } };\n" % (name, name))
        for T, S in TYPES:
            o.entry("%s_%s_12" % (name, S), "void",
                    [("int", "n"), (T + "*", "x"), ("int", "sx"), ("int", "nx"), (T + "*", "y"), ("int", "sy"), ("int", "ny"), (T + "*", "z")],
                    "launch_bcast12<%s>(stream, n, x, sx, nx, y, sy, ny, z, Op2_%s<%s>())" % (T, name, T), "src/libknet8/cuda12.jl:18-34")
            p13 = [(T + "*", "x"), (T + "*", "y"), (T + "*", "z"), ("int", "dimstride"), ("int", "nextstride"), ("int", "multidimsize"),
                   ("int", "A_N"), ("int", "B_N")]
            o.entry("%s_%s_13_x_y" % (name, S), "void", p13,
                    "(void)nextstride; (void)multidimsize; launch_bcast12<%s>(stream, A_N, x, 1, A_N, y, dimstride, B_N, z, Op2_%s<%s>())" % (T, name, T),
                    "src/libknet8/cuda13.jl:44-106")
            o.entry("%s_%s_13_y_x" % (name, S), "void", p13,
                    "(void)nextstride; (void)multidimsize; launch_bcast12<%s>(stream, A_N, x, 1, A_N, y, dimstride, B_N, z, Op2r_%s<%s>())" % (T, name, T),
                    "src/libknet8/cuda13.jl:108-184")
    o.decl.append("\n/* ---- general N-d broadcast: element strides per dimension, 0 for a broadcast dimension; z contiguous with N elements.\n"
                  "   _16_3/_16_4/_16_5 take the strides by value (src/libknet8/cuda16.jl:10-88), _17 in device int arrays of length\n"
                  "   dimlen_z (src/libknet8/cuda17.jl:25-64); caller src/knetarrays/binary.jl:96-125 ---- */")
    for name, body, cite in ALL_BINARY_OPS:
        for T, S in TYPES:
            for nd in (3, 4, 5):
                ps = [(T + "*", "x"), (T + "*", "y"), (T + "*", "z")]
                for arr in ("x", "y", "z"):
                    ps += [("int", "stride_%s%d" % (arr, k + 1)) for k in range(nd)]
                ps.append(("int", "N_z"))
                arrs = "; ".join("const int s%s[%d] = {%s}" % (arr, nd, ", ".join("stride_%s%d" % (arr, k + 1) for k in range(nd))) for arr in ("x", "y", "z"))
                o.entry("%s_%s_16_%d" % (name, S, nd), "void", ps, None, "src/libknet8/cuda16.jl:60-86",
                        body="  %s;\n  launch_bcast_nd<%s>(stream, %d, sx, sy, sz, N_z, x, y, z, Op2_%s<%s>());\n  knet8::check_launch(\"%s_%s_16_%d\");"
                             % (arrs, T, nd, name, T, name, S, nd))
            o.entry("%s_%s_17" % (name, S), "void",
                    [(T + "*", "x"), (T + "*", "y"), (T + "*", "z"), ("int*", "stride_x"), ("int*", "stride_y"), ("int*", "stride_z"), ("int", "N_z"), ("int", "dimlen_z")],
                    "launch_bcast17<%s>(stream, x, y, z, stride_x, stride_y, stride_z, N_z, dimlen_z, Op2_%s<%s>())" % (T, name, T),
                    "src/libknet8/cuda17.jl:58-64")
    return o


def gen_elementwise():
    o = Out()
    s = o.src
    s.append(PRELUDE)
    o.decl.append("\n/* ---- elementwise forward: y[i] = f(x[i]) -- src/libknet8/cuda1.jl:13-38 ---- */")
    for name, body, cite in UNARY_OPS:
        s.append(functor("Op_" + name, ["xi"], body))
        for T, S in TYPES:
            o.entry("%s_%s" % (name, S), "void", [("int", "n"), (T + "*", "x"), (T + "*", "y")],
                    "launch_ew<%s, 1>(stream, n, x, (const %s*)nullptr, (const %s*)nullptr, y, Op_%s<%s>())" % (T, T, T, name, T), cite)
    # functors of every row of the binary table: Op2_NAME(xi, yi); the gradient rows keep their Op11_ names (xi = dy, yi = y)
    s.append(binary_functors())
    o.decl.append("\n/* ---- scalar (op) array: z[i] = f(xi, y[i]) -- src/libknet8/cuda01.jl:11-25 ---- */")
    for name, body, cite in ALL_BINARY_OPS:
        s.append("template <typename T> struct Op01_%s { T xi; __device__ __forceinline__ T operator()(T yi) const { return Op2_%s<T>()(xi, yi); } };\n" % (name, name))
        for T, S in TYPES:
            o.entry("%s_%s_01" % (name, S), "void", [("int", "n"), (T, "xi"), (T + "*", "y"), (T + "*", "z")],
                    "launch_ew<%s, 1>(stream, n, y, (const %s*)nullptr, (const %s*)nullptr, z, Op01_%s<%s>{xi})" % (T, T, T, name, T), cite)
    o.decl.append("\n/* ---- same-shape binary: z[i] = f(x[i], y[i]) -- src/libknet8/cuda11.jl:12-28 ---- */")
    for name, body, cite in BINARY_OPS + BACKBIN_OPS:
        for T, S in TYPES:
            o.entry("%s_%s_11" % (name, S), "void", [("int", "n"), (T + "*", "x"), (T + "*", "y"), (T + "*", "z")],
                    "launch_ew<%s, 2>(stream, n, x, y, (const %s*)nullptr, z, Op2_%s<%s>())" % (T, T, name, T), cite)
    o.decl.append("\n/* ---- unary functions with an integer degree: y[i] = f(d, x[i]) -- src/libknet8/cuda1.jl:49-79 ---- */")
    for name, fn, cite in INT_DEGREE_OPS:
        s.append("template <typename T> struct OpDeg_%s { int d; __device__ __forceinline__ T operator()(T xi) const { return %s<T>(d, xi); } };\n" % (name, fn))
        for T, S in TYPES:
            o.entry("%s_%s" % (name, S), "void", [("int", "n"), ("int", "d"), (T + "*", "x"), (T + "*", "y")],
                    "launch_ew<%s, 1>(stream, n, x, (const %s*)nullptr, (const %s*)nullptr, y, OpDeg_%s<%s>{d})" % (T, T, T, name, T), cite)
    o.decl.append("\n/* ---- activation gradients dx[i] = f(dy[i], y[i]) -- src/libknet8/cuda11.jl:12-28 with the *back rows of ops.jl:114-121 ---- */")
    for name, body, cite in BACK11_OPS:
        for T, S in TYPES:
            o.entry("%s_%s_11" % (name, S), "void", [("int", "n"), (T + "*", "dy"), (T + "*", "y"), (T + "*", "dx")],
                    "launch_ew<%s, 2>(stream, n, dy, y, (const %s*)nullptr, dx, Op11_%s<%s>())" % (T, T, name, T), cite)
    o.decl.append("\n/* ---- ops21 gradients dx[i] = f(x[i], y[i], dy[i]) -- src/libknet8/cuda111.jl:12-29 ---- */")
    for name, body, cite in BACK111_OPS:
        s.append(functor("Op111_" + name, ["x", "y", "dy"], "(void)x; (void)y; " + body))
        for T, S in TYPES:
            o.entry("%s_%s_111" % (name, S), "void", [("int", "n"), (T + "*", "x"), (T + "*", "y"), (T + "*", "dy"), (T + "*", "dx")],
                    "launch_ew<%s, 3>(stream, n, x, y, dy, dx, Op111_%s<%s>())" % (T, name, T), cite)
    o.decl.append("\n/* ---- relu with max_value / negative_slope / threshold -- src/libknet8/relu.jl:8-38, src/ops21/activation.jl:101-112 ---- */")
    s.append("template <typename T> struct OpReluKw { T maxv, slope, thr; __device__ __forceinline__ T operator()(T x) const {\n"
             "  if (x >= maxv) return maxv; if (x >= thr) return x; if (slope == T(0)) return T(0); const T a = x - thr; return slope * a; } };\n")
    s.append("template <typename T> struct OpRelubackKw { T maxv, slope, thr; __device__ __forceinline__ T operator()(T x, T dy) const {\n"
             "  const T g = x >= maxv ? T(0) : x >= thr ? T(1) : slope; return dy * g; } };\n")
    for T, S in TYPES:
        o.entry("relu_%s_1" % S, "void", [("int", "n"), (T, "max_value"), (T, "negative_slope"), (T, "threshold"), (T + "*", "x"), (T + "*", "y")],
                "launch_ew<%s, 1>(stream, n, x, (const %s*)nullptr, (const %s*)nullptr, y, OpReluKw<%s>{max_value, negative_slope, threshold})" % (T, T, T, T),
                "src/libknet8/relu.jl:8-15,26-31")
        o.entry("reluback_%s_1" % S, "void",
                [("int", "n"), (T, "max_value"), (T, "negative_slope"), (T, "threshold"), (T + "*", "x"), (T + "*", "y"), (T + "*", "dy"), (T + "*", "dx")],
                "(void)y; launch_ew<%s, 2>(stream, n, x, dy, (const %s*)nullptr, dx, OpRelubackKw<%s>{max_value, negative_slope, threshold})" % (T, T, T),
                "src/libknet8/relu.jl:17-24,32-37 (y is not read: 3 streams instead of 4)")
    o.decl.append("\n/* ---- fill, dropout, axpy, scal ---- */")
    s.append("template <typename T> struct OpFill { T v; __device__ __forceinline__ T operator()() const { return v; } };\n")
    s.append("// dropout!: y holds U[0,1) on entry; y = y>p ? x/q : 0 with q = 1-p  (src/ops20/dropout.jl:45-58)\n"
             "template <typename T> struct OpDropout { T p, q; __device__ __forceinline__ T operator()(T x, T u) const { return u > p ? x / q : T(0); } };\n")
    s.append("// dropback!: dx = y==0 ? 0 : dy/q  (src/ops20/dropout.jl:60-71)\n"
             "template <typename T> struct OpDropback { T q; __device__ __forceinline__ T operator()(T y, T dy) const { return y == T(0) ? T(0) : dy / q; } };\n")
    s.append("template <typename T> struct OpAxpy { T a; __device__ __forceinline__ T operator()(T x, T y) const { const T p = a * x; return y + p; } };\n")
    s.append("template <typename T> struct OpScal { T a; __device__ __forceinline__ T operator()(T x) const { return a * x; } };\n")
    o.decl.append("/* rand_S / randn_S: y[0..n) = U[0,1) / N(0,1) from the default stream -- what rand!(a::KnetArray) and randn! take from\n"
                  "   cuRAND (src/knetarrays/random.jl:5-6; dropout! draws its mask buffer this way, src/ops20_gpu/dropout.jl:14).  The\n"
                  "   *_seeded forms name the stream position explicitly: Philox4x32-10 with key = seed, counters offset, offset+1, ...\n"
                  "   (4 fp32 or 2 fp64 values per counter), so element i depends on (seed, offset, i) only.  Under hipGraph capture use the\n"
                  "   seeded forms: the default stream's position is read at capture time and every replay would repeat it. */")
    for T, S in TYPES:
        for name, normal in (("rand", "false"), ("randn", "true")):
            o.entry("%s_%s" % (name, S), "void", [("int", "n"), (T + "*", "y")], None, "src/knetarrays/random.jl:5-6",
                    body="  if (n <= 0) return;\n  unsigned long long seed, offset;\n  knet8::rng_take(rand_blocks<%s>(n), &seed, &offset);\n"
                         "  launch_rand<%s, %s>(stream, n, seed, offset, y);\n  knet8::check_launch(\"%s_%s\");" % (T, T, normal, name, S))
            o.entry("%s_seeded_%s" % (name, S), "void", [("int", "n"), ("unsigned long long", "seed"), ("unsigned long long", "offset"), (T + "*", "y")],
                    "launch_rand<%s, %s>(stream, n, seed, offset, y)" % (T, normal), "src/knetarrays/random.jl:5-6 with the generator state passed in")
            o.entry("%s_state_%s" % (name, S), "void", [("int", "n"), ("unsigned long long*", "state"), (T + "*", "y")],
                    "launch_rand_state<%s, %s>(stream, n, state, y)" % (T, normal),
                    "src/knetarrays/random.jl:5-6 with the generator state {seed, next counter} in device memory: read by the launch and\n"
                    "   moved forward by a second one-lane launch, so a captured graph draws fresh numbers on every replay")
    for T, S in TYPES:
        o.entry("fill_%s" % S, "void", [("int", "n"), (T, "x"), (T + "*", "y")],
                "launch_ew<%s, 0>(stream, n, (const %s*)nullptr, (const %s*)nullptr, (const %s*)nullptr, y, OpFill<%s>{x})" % (T, T, T, T, T),
                "src/libknet8/cuda1.jl:82-105")
        o.entry("dropout_%s" % S, "void", [("int", "n"), (T, "p"), (T + "*", "x"), (T + "*", "y")],
                "launch_ew<%s, 2>(stream, n, x, y, (const %s*)nullptr, y, OpDropout<%s>{p, %s(1) - p})" % (T, T, T, T),
                "src/libknet8/cuda1.jl:459-484 (in place: y is the uniform buffer on entry)")
        o.entry("dropback_%s" % S, "void", [("int", "n"), (T, "p"), (T + "*", "x"), (T + "*", "y"), (T + "*", "dy"), (T + "*", "dx")],
                "(void)x; launch_ew<%s, 2>(stream, n, y, dy, (const %s*)nullptr, dx, OpDropback<%s>{%s(1) - p})" % (T, T, T, T),
                "src/libknet8/cuda1.jl:469-493")
        o.entry("axpy_%s" % S, "void", [("int", "n"), (T, "alpha"), (T + "*", "x"), (T + "*", "y")],
                "launch_ew<%s, 2>(stream, n, x, y, (const %s*)nullptr, y, OpAxpy<%s>{alpha})" % (T, T, T),
                "cublas%saxpy_v2 with unit increments at src/knetarrays/linalg.jl:58-73 (addto!, src/autograd_gpu/addto.jl:7-10)" % ("S" if S == "32" else "D"))
        o.entry("scal_%s" % S, "void", [("int", "n"), (T, "alpha"), (T + "*", "x")],
                "launch_ew<%s, 1>(stream, n, x, (const %s*)nullptr, (const %s*)nullptr, x, OpScal<%s>{alpha})" % (T, T, T, T),
                "cublas%sscal_v2 with unit increment at src/knetarrays/linalg.jl:75-90" % ("S" if S == "32" else "D"))
    o.decl.append("\n/* ---- binary cross entropy on raw scores with {0,1} labels already converted to T (oftype(scores,labels)).  No libknet8\n"
                  "   counterpart: bce_S replaces the broadcast chain max.(0,s) .- y.*s .+ log.(1 .+ exp.(-abs.(s))) of src/ops20/loss.jl:107-111\n"
                  "   (per-element losses, to be summed); bceback_S is its gradient wrt the scores times `scale`. ---- */")
    s.append("template <typename T> struct OpBce { __device__ __forceinline__ T operator()(T sc, T y) const {\n"
             "  const T a = sc > T(0) ? sc : T(0); const T b = y * sc; const T c = a - b; const T ab = sc < T(0) ? -sc : sc;\n"
             "  const T e = kexp(-ab); const T f = T(1) + e; return c + klog(f); } };\n")
    s.append("template <typename T> struct OpBceBack { T scale; __device__ __forceinline__ T operator()(T sc, T y) const {\n"
             "  const T ab = sc < T(0) ? -sc : sc; const T e = kexp(-ab); const T q = e / (T(1) + e);\n"
             "  const T step = sc > T(0) ? T(1) : T(0); const T sg = sc > T(0) ? T(1) : sc < T(0) ? T(-1) : T(0);\n"
             "  const T g = (step - y) - sg * q; return scale * g; } };\n")
    for T, S in TYPES:
        o.entry("bce_%s" % S, "void", [("int", "n"), (T + "*", "scores"), (T + "*", "labels"), (T + "*", "loss")],
                "launch_ew<%s, 2>(stream, n, scores, labels, (const %s*)nullptr, loss, OpBce<%s>())" % (T, T, T), "src/ops20/loss.jl:107-111")
        o.entry("bceback_%s" % S, "void", [("int", "n"), (T, "scale"), (T + "*", "scores"), (T + "*", "labels"), (T + "*", "dscores")],
                "launch_ew<%s, 2>(stream, n, scores, labels, (const %s*)nullptr, dscores, OpBceBack<%s>{scale})" % (T, T, T),
                "the AutoGrad gradient of the same chain (max, abs, exp, log rules), src/ops20/loss.jl:107-111")
    o.decl.append("\n/* ---- fused optimizer updates (in place).  No libknet8 counterpart: each replaces the lmul!/axpy!/broadcast chain of one\n"
                  "   _update! method of src/train20/update.jl:513-570 (SGD itself is axpy_S).  Scalars are the T-rounded constants the\n"
                  "   Julia code forms: nlr = T(-lr), opg = T(1+gamma), omr = T(1-rho), omb1 = T(1-beta1), c1 = T(1-beta1^t) ... ---- */")
    for name, scalars, arrays, mask, body, cite in OPTIMIZER_OPS:
        fields = " ".join("T %s;" % x for x in scalars)
        s.append("template <typename T> struct Opt_%s { %s __device__ __forceinline__ void operator()(T (&v)[%d]) const { %s } };\n"
                 % (name, fields, len(arrays), body))
        for T, S in TYPES:
            params = [("int", "n")] + [(T, x) for x in scalars] + [(T + "*", a) for a in arrays]
            ptrs = arrays + ["(%s*)nullptr" % T] * (4 - len(arrays))
            o.entry("%s_%s" % (name, S), "void", params,
                    "launch_update<%s, %d, %du>(stream, n, %s, Opt_%s<%s>{%s})" % (T, len(arrays), mask, ", ".join(ptrs), name, T, ", ".join(scalars)), cite)
    o.decl.append("\n/* ---- fused dense-layer passes on an m x n column-major matrix with bias b of shape (m,1).  No libknet8 counterpart:\n"
                  "   biasF_S replaces add_S_12 followed by F_S (src/knetarrays/binary.jl:61-95, src/ops20_gpu/activation.jl:17-29);\n"
                  "   biasreludrop_S also applies dropout! with y holding U[0,1) on entry (src/ops20/dropout.jl:45-58);\n"
                  "   Fback_biasgrad_S replaces Fback_S_11 followed by sum(dz;dims=2) (src/ops20_gpu/activation.jl:30-37,\n"
                  "   src/knetarrays/reduction.jl:21-77); dropreluback_biasgrad_S starts from the dropout output (dropback!,\n"
                  "   src/ops20/dropout.jl:60-71).  y and dz carry the same bits as the separate launches. ---- */")
    s.append("template <typename T, typename Op> struct BiasAct { __device__ __forceinline__ T operator()(T zb, T) const { return Op()(zb); } };\n")
    s.append("template <typename T> struct BiasReluDrop { T p, q; __device__ __forceinline__ T operator()(T zb, T u) const {\n"
             "  const T r = Op_relu<T>()(zb); return u > p ? r / q : T(0); } };\n")
    s.append("// dropback! then reluback from the dropout output alone: the output is positive exactly where the element was kept and the relu active\n"
             "template <typename T> struct OpDropReluBack { T q; __device__ __forceinline__ T operator()(T dy, T y) const { return y > T(0) ? dy / q : T(0); } };\n")
    for act in FUSED_ACTS:
        for T, S in TYPES:
            o.entry("bias%s_%s" % (act, S), "void", [("int", "m"), ("int", "n"), (T + "*", "z"), (T + "*", "b"), (T + "*", "y")],
                    "launch_bias_act<%s, false>(stream, m, n, z, b, y, BiasAct<%s, Op_%s<%s> >())" % (T, T, act, T),
                    "add_S_12 + %s_S, src/knetarrays/binary.jl:61-95, src/ops20_gpu/activation.jl:17-29" % act)
            o.entry("%sback_biasgrad_%s" % (act, S), "void",
                    [("int", "m"), ("int", "n"), (T + "*", "dy"), (T + "*", "y"), (T + "*", "dz"), (T + "*", "db")],
                    "launch_actback_biasgrad<%s>(stream, m, n, dy, y, dz, db, Op11_%sback<%s>())" % (T, act, T),
                    "%sback_S_11 + sum_S_21, src/ops20_gpu/activation.jl:30-37, src/knetarrays/reduction.jl:21-77" % act)
    o.decl.append("/* dense_back_S: the backward pass of one small dense layer y = f(W*x + b) in one launch.  W is m x k, x is k x n, y and dy\n"
                  "   are m x n (column-major, no padding); act 0: dz = dy, act 1: dz = y > 0 ? dy : 0 (relu).  Writes dW = dz*x' (m x k),\n"
                  "   db = sum(dz; dims=2) (m) and dx = W'*dz (k x n); any of the three may be NULL (db needs dW).  Returns 0 when done, 1 when\n"
                  "   the layer is too large for the small-matrix kernels -- nothing is launched then and the caller uses Fback_biasgrad_S\n"
                  "   and gemm_S instead --, -1 on bad arguments.  No libknet8 counterpart: replaces reluback + sum(dz;dims=2) + two gemm!\n"
                  "   calls (src/ops20_gpu/activation.jl:30-37, src/knetarrays/reduction.jl:21-77, src/knetarrays/linalg.jl:11-18). */")
    for T, S in TYPES:
        o.entry("dense_back_%s" % S, "int",
                [("int", "act"), ("int", "m"), ("int", "n"), ("int", "k"), (T + "*", "W"), (T + "*", "x"), (T + "*", "y"), (T + "*", "dy"),
                 (T + "*", "dW"), (T + "*", "db"), (T + "*", "dx")], None,
                "reluback_S_11 + sum_S_21 + gemm! x 2, src/knetarrays/linalg.jl:11-18",
                body="  const int rc = launch_dense_back<%s>(stream, act, m, n, k, W, x, y, dy, dW, db, dx);\n  knet8::check_launch(\"dense_back_%s\");\n  return rc;" % (T, S))
    o.decl.append("/* dense_nll_back_S: backward pass of a classifier's output layer with the loss folded in.  z = W*x + b are the scores (m classes x n\n"
                  "   instances, m <= 16), labels 1-based int32 (0 skips the instance).  Writes loss[j] = -logsoftmax(z)[label_j, j], mean[0] =\n"
                  "   scale * sum(loss) (the average loss when scale = 1/count) and, with dz = scale*(softmax(z) - onehot(label)): dW = dz*x' (m x k),\n"
                  "   db = sum(dz; dims=2), dx = W'*dz (k x n); dW, db, dx, loss, mean may be NULL (db, loss and mean need dW).  Returns 0 when done, 1 when not applicable (more than 16 classes, or too large: nothing is launched and\n"
                  "   the caller uses nll_logsoftmax_back_S + dense_back_S), -1 on bad arguments.  No libknet8 counterpart: replaces the chain of\n"
                  "   src/ops20/loss.jl:37-41 plus sum(dz;dims=2) and two gemm! calls (src/knetarrays/linalg.jl:11-18). */")
    for T, S in TYPES:
        o.entry("dense_nll_back_%s" % S, "int",
                [("int", "m"), ("int", "n"), ("int", "k"), (T + "*", "W"), (T + "*", "x"), (T + "*", "z"), ("int*", "labels"), (T, "scale"),
                 (T + "*", "dW"), (T + "*", "db"), (T + "*", "dx"), (T + "*", "loss"), (T + "*", "mean")], None,
                "nll -> logsoftmax -> getindex (src/ops20/loss.jl:37-41) + sum_S_21 + gemm! x 2, src/knetarrays/linalg.jl:11-18",
                body="  const int rc = launch_dense_nll_back<%s>(stream, m, n, k, W, x, z, labels, scale, dW, db, dx, loss, mean);\n  knet8::check_launch(\"dense_nll_back_%s\");\n  return rc;" % (T, S))
    o.decl.append("/* dense_head_S: a classifier's output layer forward and backward in one launch.  From W (m x k), bias (m), the layer's input x (k x n)\n"
                  "   and the labels: the scores z = W*x + bias (written to z when z is not NULL), and everything dense_nll_back_S writes from them\n"
                  "   (loss, mean, dW, db, dx).  m <= 16 classes, n <= 512 instances (fp64: 256), dW required; returns 0 when done, 1 when not applicable\n"
                  "   (nothing launched: use gemm_bias_act_S + dense_nll_back_S), -1 on bad arguments.  No libknet8 counterpart. */")
    for T, S in TYPES:
        o.entry("dense_head_%s" % S, "int",
                [("int", "m"), ("int", "n"), ("int", "k"), (T + "*", "W"), (T + "*", "bias"), (T + "*", "x"), ("int*", "labels"), (T, "scale"),
                 (T + "*", "dW"), (T + "*", "db"), (T + "*", "dx"), (T + "*", "loss"), (T + "*", "mean"), (T + "*", "z")], None,
                "gemm! + bias broadcast (src/knetarrays/linalg.jl:26-52, binary.jl:61-95) + the chain of src/ops20/loss.jl:37-41 + sum_S_21 + gemm! x 2",
                body="  const int rc = launch_dense_head<%s>(stream, m, n, k, W, bias, x, labels, scale, dW, db, dx, loss, mean, z);\n  knet8::check_launch(\"dense_head_%s\");\n  return rc;" % (T, S))
    for T, S in TYPES:
        o.entry("biasreludrop_%s" % S, "void", [("int", "m"), ("int", "n"), (T, "p"), (T + "*", "z"), (T + "*", "b"), (T + "*", "y")],
                "launch_bias_act<%s, true>(stream, m, n, z, b, y, BiasReluDrop<%s>{p, %s(1) - p})" % (T, T, T),
                "add_S_12 + relu_S + dropout_S, src/ops20/dropout.jl:45-58")
        o.entry("dropreluback_biasgrad_%s" % S, "void",
                [("int", "m"), ("int", "n"), (T, "p"), (T + "*", "dy"), (T + "*", "y"), (T + "*", "dz"), (T + "*", "db")],
                "launch_actback_biasgrad<%s>(stream, m, n, dy, y, dz, db, OpDropReluBack<%s>{%s(1) - p})" % (T, T, T),
                "dropback_S + reluback_S_11 + sum_S_21, src/ops20/dropout.jl:60-71")
    return o


def gen_reduce():
    o = Out()
    o.src.append(PRELUDE)
    o.decl.append("\n/* ---- reductions.  _20: whole array -> scalar returned by value (blocks until done);\n"
                  "   _21: x[i] goes into y[(i/sy)%ny]; _22: N-d array, one reduced dim of size xd1+1 and stride s1,\n"
                  "   next stride s2 -- src/libknet8/cuda20.jl:27-104, cuda21.jl:22-77, cuda22.jl:22-66;\n"
                  "   dispatch src/knetarrays/reduction.jl:21-77 ---- */")
    for name, cls in REDUCTION_OPS:
        for T, S in TYPES:
            op = "%s<%s>" % (cls, T)
            body20 = ("  %s r = %s::init();\n"
                      "  if (n <= 0) return r;\n"
                      "  %s* out = static_cast<%s*>(knet8::scalar_slot(stream));\n"
                      "  launch_reduce_run<%s, %s>(stream, x, (long)n, 1, 1, out);\n"
                      "  knet8::check_launch(\"%s_%s_20\");\n"
                      "  knet8::fetch_scalar(stream, out, &r, sizeof(r));\n"
                      "  return r;") % (T, op, T, T, T, op, name, S)
            o.entry("%s_%s_20" % (name, S), T, [("int", "n"), (T + "*", "x")], None, "src/libknet8/cuda20.jl:84-104", body=body20)
            o.entry("%s_%s_21" % (name, S), "void", [("int", "nx"), (T + "*", "x"), ("int", "sy"), ("int", "ny"), (T + "*", "y")],
                    "knet8::reduce_21<%s, %s>(stream, nx, x, sy, ny, y)" % (T, op), "src/libknet8/cuda21.jl:68-76")
            o.entry("%s_%s_22" % (name, S), "void",
                    [("int", "nx"), ("int", "xd1"), (T + "*", "x"), ("int", "s1"), ("int", "s2"), ("int", "ny"), (T + "*", "y")],
                    "knet8::reduce_22<%s, %s>(stream, nx, xd1, x, s1, s2, ny, y)" % (T, op), "src/libknet8/cuda22.jl:58-65")
    return o


def gen_softmax():
    o = Out()
    o.src.append(PRELUDE)
    o.decl.append("\n/* ---- softmax family down each contiguous column of an m x n column-major matrix.  No libknet8 counterpart:\n"
                  "   these replace the cudnnSoftmaxForward/Backward calls (MODE_INSTANCE on a (1,1,m,n) view, ACCURATE and LOG\n"
                  "   algorithms) at src/ops20_gpu/softmax.jl:44-56; arithmetic of src/ops20/softmax.jl:42-63 ---- */")
    for T, S in TYPES:
        z = "(const %s*)nullptr" % T
        o.entry("softmax_%s" % S, "void", [("int", "m"), ("int", "n"), (T + "*", "x"), (T + "*", "y")],
                "launch_softmax<%s, AlgoSoftmax<%s>>(stream, m, n, x, %s, y, nullptr, %s(0), nullptr)" % (T, T, z, T),
                "unsafe_cudnnSoftmaxForward(ACCURATE) at src/ops20_gpu/softmax.jl:44-49")
        o.entry("logsoftmax_%s" % S, "void", [("int", "m"), ("int", "n"), (T + "*", "x"), (T + "*", "y")],
                "launch_softmax<%s, AlgoLogSoftmax<%s>>(stream, m, n, x, %s, y, nullptr, %s(0), nullptr)" % (T, T, z, T),
                "unsafe_cudnnSoftmaxForward(LOG) at src/ops20_gpu/softmax.jl:44-49")
        o.entry("softmaxback_%s" % S, "void", [("int", "m"), ("int", "n"), (T + "*", "y"), (T + "*", "dy"), (T + "*", "dx")],
                "launch_softmax<%s, AlgoSoftmaxBack<%s>>(stream, m, n, y, dy, dx, nullptr, %s(0), nullptr)" % (T, T, T),
                "unsafe_cudnnSoftmaxBackward(ACCURATE) at src/ops20_gpu/softmax.jl:51-56")
        o.entry("logsoftmaxback_%s" % S, "void", [("int", "m"), ("int", "n"), (T + "*", "y"), (T + "*", "dy"), (T + "*", "dx")],
                "launch_softmax<%s, AlgoLogSoftmaxBack<%s>>(stream, m, n, y, dy, dx, nullptr, %s(0), nullptr)" % (T, T, T),
                "unsafe_cudnnSoftmaxBackward(LOG) at src/ops20_gpu/softmax.jl:51-56")
        o.decl.append("/* The same four operations along the middle axis of an (inner, d, outer) column-major view (inner > 1): softmax over a\n"
                      "   non-leading dimension, which the reference builds from broadcast and reduction kernels (src/ops20_gpu/softmax.jl:22). */")
        for nm, algo, two in (("softmax", "AlgoSoftmax", False), ("logsoftmax", "AlgoLogSoftmax", False),
                              ("softmaxback", "AlgoSoftmaxBack", True), ("logsoftmaxback", "AlgoLogSoftmaxBack", True)):
            params = [("int", "inner"), ("int", "d"), ("int", "outer")] + ([(T + "*", "y"), (T + "*", "dy"), (T + "*", "dx")] if two else [(T + "*", "x"), (T + "*", "y")])
            call = ("launch_softmax_strided<%s, %s<%s>>(stream, inner, d, outer, y, dy, dx)" % (T, algo, T)) if two else \
                   ("launch_softmax_strided<%s, %s<%s>>(stream, inner, d, outer, x, %s, y)" % (T, algo, T, z))
            o.entry("%s_strided_%s" % (nm, S), "void", params, call, "the generic _softmax/_logsoftmax path of src/ops20/softmax.jl:42-63 for dims that are not leading")
        o.decl.append("/* Fused gradient of nll(scores, labels; dims=1) wrt scores: dx = scale*(softmax(x) - onehot(label)) per column and\n"
                      "   loss[col] = -logsoftmax(x)[label, col]; labels are 1-based int32, label 0 skips the column (dx = 0, loss = 0).\n"
                      "   One pass over the scores instead of logsoftmax + getents + fill + addents + logsoftmaxback. */")
        o.entry("nll_logsoftmax_back_%s" % S, "void",
                [("int", "m"), ("int", "n"), (T + "*", "scores"), ("int*", "labels"), (T, "scale"), (T + "*", "dx"), (T + "*", "loss")],
                "launch_softmax<%s, AlgoNll<%s>>(stream, m, n, scores, %s, dx, labels, scale, loss)" % (T, T, z),
                "the chain nll -> getindex -> logsoftmax of src/ops20/loss.jl:37-41 (getents/addents + cuDNN LOG backward)")
    o.decl.append("\n/* ---- 2-d transpose y(n,m) = x(m,n)' -- CUDA.jl permutedims / cublasSgeam at src/knetarrays/reshape.jl:18, linalg.jl:92-113 ---- */")
    for T, S in TYPES:
        o.entry("transpose_%s" % S, "void", [("int", "m"), ("int", "n"), (T + "*", "x"), (T + "*", "y")],
                "launch_transpose<%s>(stream, m, n, x, y)" % T, "permutedims(x) for matrices, src/ops20_gpu/softmax.jl:19-20")
        o.entry("permute213_%s" % S, "void", [("int", "m"), ("int", "n"), ("int", "batch"), (T + "*", "x"), (T + "*", "y")],
                "launch_transpose<%s>(stream, m, n, x, y, batch)" % T,
                "permutedims(x, (2,1,3)) of an (m, n, batch) array (CUDA.jl's permutedims in the reference, src/knetarrays/reshape.jl:18)")
    o.decl.append("/* permutedims_S: y = permutedims(x, perm) for an array of `ndims` (1 to 8) dimensions.  `dims` (sizes of x) and `perm`\n"
                  "   (1-based, as in Julia) are HOST arrays read during the call; x and y are device arrays of prod(dims) elements.\n"
                  "   Replaces permutedims!(CuArray(y), CuArray(x), perm) of CUDA.jl at src/knetarrays/reshape.jl:18-29. */")
    for T, S in TYPES:
        o.entry("permutedims_%s" % S, "void", [("int", "ndims"), ("const int*", "dims"), ("const int*", "perm"), (T + "*", "x"), (T + "*", "y")],
                "launch_permutedims<%s>(stream, ndims, dims, perm, x, y)" % T, "src/knetarrays/reshape.jl:18-29")
    o.decl.append("\n/* ---- gather / scatter on 1-based int32 linear indices -- src/libknet8/cuda1.jl:342-362 ---- */")
    for T, S in TYPES:
        o.entry("getents_%s" % S, "void", [("int", "n"), ("int*", "ents"), (T + "*", "x"), (T + "*", "y")],
                "launch_getents<%s>(stream, n, ents, x, y)" % T, "src/libknet8/cuda1.jl:342-348")
        o.entry("setents_%s" % S, "void", [("int", "n"), ("int*", "ents"), (T + "*", "x"), (T + "*", "y")],
                "launch_setents<%s>(stream, n, ents, x, y)" % T, "src/libknet8/cuda1.jl:349-355")
        o.entry("addents_%s" % S, "void", [("int", "n"), ("int*", "ents"), (T + "*", "x"), (T + "*", "y")],
                "launch_addents<%s>(stream, n, ents, x, y)" % T, "src/libknet8/cuda1.jl:356-362")
        o.entry("setent1_%s" % S, "void", [("int", "n"), ("int*", "ents"), (T + "*", "x"), (T, "y")],
                "launch_setent1<%s>(stream, n, ents, x, y)" % T, "src/libknet8/cuda1.jl:363-369")
    o.decl.append("\n/* ---- whole columns / rows of an xrows x xcols matrix by 1-based int32 index: get (y = x[sel]), set (x[sel] = y), add (x[sel] += y,\n"
                  "   atomic: repeated indices accumulate), set1 (x[sel] = scalar) -- src/libknet8/cuda1.jl:234-341 ---- */")
    for T, S in TYPES:
        for kind, sel, n in (("cols", "cols", "ncols"), ("rows", "rows", "nrows")):
            one = kind[:-1] + "1"
            for mode, name in enumerate(("get" + kind, "set" + kind, "add" + kind)):
                o.entry("%s_%s" % (name, S), "void", [("int", "xrows"), ("int", "xcols"), ("int", n), ("int*", sel), (T + "*", "x"), (T + "*", "y")],
                        "launch_%s<%s, %d>(stream, xrows, xcols, %s, %s, x, y, %s(0))" % (kind, T, mode, n, sel, T), "src/libknet8/cuda1.jl:234-341")
            o.entry("set%s_%s" % (one, S), "void", [("int", "xrows"), ("int", "xcols"), ("int", n), ("int*", sel), (T + "*", "x"), (T, "y")],
                    "launch_%s<%s, 3>(stream, xrows, xcols, %s, %s, x, (%s*)nullptr, y)" % (kind, T, n, sel, T), "src/libknet8/cuda1.jl:234-341")
    o.decl.append("\n/* ---- rectangular blocks and concatenation.  xcopy counts rows and steps in BYTES, xfill in elements; icat takes a HOST array of\n"
                  "   device pointers, concat device arrays of starts, lengths and pointers -- src/libknet8/cuda1.jl:107-207,503-530 ---- */")
    o.entry("xcopy", "void", [("int", "nrows"), ("int", "ncols"), ("const void*", "x"), ("int", "incx"), ("void*", "y"), ("int", "incy")],
            "launch_xcopy(stream, nrows, ncols, x, incx, y, incy)", "src/libknet8/cuda1.jl:130-165")
    for T, S in TYPES:
        o.entry("xfill_%s" % S, "void", [("int", "nrows"), ("int", "ncols"), (T, "x"), (T + "*", "y"), ("int", "incy")],
                "launch_xfill<%s>(stream, nrows, ncols, x, y, incy)" % T, "src/libknet8/cuda1.jl:107-128")
        o.entry("icat_%s" % S, "void", [("int", "nrows"), ("int", "ncols"), (T + "**", "x"), (T + "*", "y")],
                "launch_icat<%s>(stream, nrows, ncols, x, y)" % T, "src/libknet8/cuda1.jl:167-207")
        o.entry("concat_%s" % S, "void", [("int", "narrays"), ("int*", "starts"), ("int*", "lengths"), (T + "**", "x"), (T + "*", "y")],
                "launch_concat<%s>(stream, narrays, starts, lengths, x, y)" % T, "src/libknet8/cuda1.jl:503-530")
    return o


HEADER_TOP = """/* knet8.h -- C ABI of libknet8.so for AMD Instinct MI355X (gfx950).
 *
 * GENERATED by knet.jl_amd/csrc/gen_knet8.py together with the sources of the library.
 *
 * Every kernel entry point exists twice, as in the reference (src/libknet8/LibKnet8.jl:50-62):
 *   NAME_stream(args..., hipStream_t)  -- asynchronous launch on the given stream (what @knet8 binds)
 *   NAME(args...)                      -- same on the null stream
 * S in a name is the element width (32: float, 64: double).  Sizes and strides are 32-bit ints, scalars
 * are passed by value in T, arrays are device pointers owned and pre-allocated by the caller, index
 * arrays hold 1-based int32.  Calls return nothing (only the _20 reductions return a value, and block);
 * n <= 0 is a no-op.  Failures are recorded and can be read with knet8_last_error().
 */
#ifndef KNET8_H
#define KNET8_H
#include <stddef.h>
#ifdef __cplusplus
extern "C" {
#endif
#ifndef KNET8_API
#define KNET8_API __attribute__((visibility("default")))
#endif
typedef struct ihipStream_t* hipStream_t;
"""

HEADER_RUNTIME = """
/* ---- runtime: device memory for KnetArray storage, copies, streams, GEMM ---- */
/* replaces knetMalloc / the free-list pool of src/knetarrays/kptr.jl:105-142,186-194: size-class pool over hipMalloc.
 * The pool knows nothing of streams, as the reference's does not: a block handed back by knet8_free may be handed out again at once, so free a block
 * only when the work that uses it was queued on the stream that its next user will queue on too (one stream per pool user), or after knet8_synchronize. */
KNET8_API void* knet8_malloc(size_t nbytes);
KNET8_API void knet8_free(void* ptr);
/* replaces Knet.gc, src/knetarrays/kptr.jl:204-226: waits for the device, then gives back every cached block of the pool, the scratch the
   library keeps per stream for split reductions (current and outgrown buffers) and its hipBLASLt workspaces -- except scratch and workspaces that
   were handed out while their stream was being captured, which a graph may still name; returns the bytes released */
KNET8_API size_t knet8_trim(void);
/* replaces meminfo/kmeminfo, src/knetarrays/kptr.jl:254-255: out[0]=bytes in use, out[1]=bytes cached, out[2]=hipMalloc calls, out[3]=pool hits */
KNET8_API void knet8_meminfo(size_t* out4);
/* no counterpart in the reference: out[0] = hipMalloc calls and out[1] = hipFree calls the library has made so far (pool, scratch, workspaces: every
   one is counted), out[2] = bytes it currently holds outside the pool (per-stream reduction scratch, hipBLASLt workspaces, the 256-byte slots of
   the _20 reductions), out[3] = plain products that ran on the library's own tiles because hipBLASLt reported no algorithm, out[4] = free and
   out[5] = total device memory in bytes (hipMemGetInfo) */
KNET8_API void knet8_stats(unsigned long long* out6);
/* replaces the copyto!/unsafe_copyto! paths of src/knetarrays/copy.jl:6-11: kind 1 = host->device, 2 = device->host, 3 = device->device;
   host copies return when the data has landed */
KNET8_API int knet8_memcpy(void* dst, const void* src, size_t nbytes, int kind, hipStream_t stream);
KNET8_API int knet8_device_count(void);
KNET8_API int knet8_set_device(int dev);
/* non-blocking streams; destroying one waits for its work and frees the reduction scratch and the hipBLASLt workspace the library keeps
   for it (destroy graphs captured on it first) */
KNET8_API hipStream_t knet8_stream_create(void);
KNET8_API void knet8_stream_destroy(hipStream_t stream);
KNET8_API int knet8_synchronize(hipStream_t stream);
/* elapsed device time between two marks on a stream, in milliseconds (HIP events) */
KNET8_API void knet8_timer_start(hipStream_t stream);
KNET8_API float knet8_timer_stop(hipStream_t stream);
/* HIP events for timing individual launches on the stream they are issued to; elapsed is in milliseconds and waits for `stop` */
KNET8_API void* knet8_event_create(void);
KNET8_API void knet8_event_destroy(void* event);
KNET8_API void knet8_event_record(void* event, hipStream_t stream);
KNET8_API float knet8_event_elapsed(void* start, void* stop);
/* hipGraph capture of a sequence of launches on a caller-created stream (no counterpart in the reference; for launch-bound
   steps such as the MNIST MLP).  The sequence must have run once eagerly on that stream first; begin/end bracket the calls to
   record, end returns an executable graph (NULL on failure), launch replays it. */
KNET8_API int knet8_graph_begin(hipStream_t stream);
KNET8_API void* knet8_graph_end(hipStream_t stream);
KNET8_API int knet8_graph_launch(void* graph, hipStream_t stream);
KNET8_API void knet8_graph_destroy(void* graph);
/* last recorded failure as text (NULL if none); reading clears it */
KNET8_API const char* knet8_last_error(void);
KNET8_API int knet8_version(void);
/* hash of the sources the binary was built from (csrc headers and .hip files, the generator, the build script), baked in by build.py:
   a loader compares it with the working tree and refuses a stale library */
KNET8_API const char* knet8_build_id(void);
/* No counterpart in the reference.  sum_32_21 for callers that cannot allocate device memory -- code under hipGraph capture, tight
   serving loops, harnesses that forbid hipMalloc: the same kernels and the same result, bit for bit (except where a launch plan would not fit the fixed array and the planner takes another: then
   to the 1e-5 of any reduction), with the partial results and
   tickets of a split launch in a fixed array inside the library (1 MiB of partials + 64 KiB of tickets per GPU, held until the process
   ends) instead of the per-stream buffers that sum_32_21 grows through hipMalloc.  Calls no hipMalloc, hipFree or other allocating
   routine.  A shape whose split needs more than the array holds is refused: the error is recorded and y is left untouched.  All calls
   on one GPU share the array, so calls that overlap in time on one GPU (other streams, other threads) race; calls on one stream are
   ordered and safe. */
KNET8_API void sum_32_21_noalloc(int nx, float* x, int sy, int ny, float* y, hipStream_t stream);
/* launch-heuristic knobs; returns the old value; value 0 restores the default, a negative value only reads.  Key 0: number of compute units the reduction planner aims at (default: asked from the
   device); key 1: longest softmax column kept resident in registers, longer ones take the two-pass streaming kernel (default 0: the register capacity);
   key 3: products of up to this many MFLOP (2*m*n*k/1e6) take the library's own small-product kernels instead of hipBLASLt (default 0: off,
   every product of gemm_S / gemm_bias_act_S goes to hipBLASLt);
   key 4: dense_back_S / dense_nll_back_S accept layers whose products have up to this many MFLOP each (default 270);
   key 5: non-zero makes the library behave as if the scratch memory of split launches could not be allocated (for tests of that error path);
   key 6: non-zero keeps softmax columns of 128 to 256 KB in registers alone instead of registers + LDS (for comparisons);
   key 7: non-zero makes the hipBLASLt route of gemm_S do everything but the vendor call itself (for measuring the library's own share of a call's host time);
   key 8: non-zero keeps repeated products on hipblasLtMatmul instead of the prepared calls of the vendor's extension interface (for comparisons) */
KNET8_API int knet8_tune(int key, int value);
/* Seed of the default random stream used by rand_S / randn_S (restarts it at counter 0): the device half of Knet.seed!,
   src/knetarrays/random.jl:14-18 (CUDA.seed!).  Unseeded, the stream starts from the operating system's entropy. */
KNET8_API void knet8_seed(unsigned long long seed);
/* replaces cublasSgemm_v2 / cublasDgemm_v2 at src/knetarrays/linalg.jl:26-52 (column-major, transa/transb in 'N','T'): hipBLASLt */
KNET8_API int gemm_32_stream(char transa, char transb, int m, int n, int k, float alpha, float* A, int lda, float* B, int ldb, float beta, float* C, int ldc, hipStream_t stream);
KNET8_API int gemm_32(char transa, char transb, int m, int n, int k, float alpha, float* A, int lda, float* B, int ldb, float beta, float* C, int ldc);
KNET8_API int gemm_64_stream(char transa, char transb, int m, int n, int k, double alpha, double* A, int lda, double* B, int ldb, double beta, double* C, int ldc, hipStream_t stream);
KNET8_API int gemm_64(char transa, char transb, int m, int n, int k, double alpha, double* A, int lda, double* B, int ldb, double beta, double* C, int ldc);
/* replaces cublasSgemmStridedBatched / cublasDgemmStridedBatched at src/ops20_gpu/bmm.jl:46-50 (bmm!): product b of the batch uses
   A + b*strideA, B + b*strideB, C + b*strideC (strides in elements); hipBLASLt strided batch */
KNET8_API int bmm_32_stream(char transa, char transb, int m, int n, int k, float alpha, float* A, int lda, long long strideA, float* B, int ldb, long long strideB, float beta, float* C, int ldc, long long strideC, int batch, hipStream_t stream);
KNET8_API int bmm_32(char transa, char transb, int m, int n, int k, float alpha, float* A, int lda, long long strideA, float* B, int ldb, long long strideB, float beta, float* C, int ldc, long long strideC, int batch);
KNET8_API int bmm_64_stream(char transa, char transb, int m, int n, int k, double alpha, double* A, int lda, long long strideA, double* B, int ldb, long long strideB, double beta, double* C, int ldc, long long strideC, int batch, hipStream_t stream);
KNET8_API int bmm_64(char transa, char transb, int m, int n, int k, double alpha, double* A, int lda, long long strideA, double* B, int ldb, long long strideB, double beta, double* C, int ldc, long long strideC, int batch);
/* dense layer in one call: C = act(alpha*op(A)*op(B) + bias[i]) with bias of length m and act 0 (none) or 1 (relu).  No counterpart in
   the reference, which runs gemm!, the bias broadcast (src/knetarrays/binary.jl:61-95) and relu (src/ops20_gpu/activation.jl:17-29) as
   three launches.  Bias and relu run in the output stage of the hipBLASLt product (its BIAS / RELU_BIAS epilogues), so the result is
   written once; where hipBLASLt has no such kernel the product is followed by one in-place pass.  The relu here is z > 0 ? z : 0 on every
   route -- the vendor epilogue's and the reference's device relu (src/libknet8/ops.jl:63): a NaN in the product comes out as 0, +Inf stays,
   -Inf becomes 0 -- whereas relu_S follows the CPU path and keeps a NaN. */
KNET8_API int gemm_bias_act_32_stream(char transa, char transb, int m, int n, int k, float alpha, float* A, int lda, float* B, int ldb, float* bias, int act, float* C, int ldc, hipStream_t stream);
KNET8_API int gemm_bias_act_32(char transa, char transb, int m, int n, int k, float alpha, float* A, int lda, float* B, int ldb, float* bias, int act, float* C, int ldc);
KNET8_API int gemm_bias_act_64_stream(char transa, char transb, int m, int n, int k, double alpha, double* A, int lda, double* B, int ldb, double* bias, int act, double* C, int ldc, hipStream_t stream);
KNET8_API int gemm_bias_act_64(char transa, char transb, int m, int n, int k, double alpha, double* A, int lda, double* B, int ldb, double* bias, int act, double* C, int ldc);
"""

HEADER_BOTTOM = """
#ifdef __cplusplus
}
#endif
#endif /* KNET8_H */
"""


def generate(write=True):
    units = {"knet8_elementwise_gen.hip": gen_elementwise(), "knet8_broadcast_gen.hip": gen_broadcast(), "knet8_reduce_gen.hip": gen_reduce(), "knet8_softmax_gen.hip": gen_softmax()}
    files = {}
    for fn, o in units.items():
        files[os.path.join(GEN, fn)] = "\n".join(o.src) + "\n"
    header = HEADER_TOP + "\n".join("\n".join(o.decl) for o in units.values()) + "\n" + HEADER_RUNTIME + HEADER_BOTTOM
    files[HEADER] = header
    if write:
        os.makedirs(GEN, exist_ok=True)
        os.makedirs(os.path.dirname(HEADER), exist_ok=True)
        for path, text in files.items():
            old = open(path).read() if os.path.exists(path) else None
            if old != text:
                with open(path, "w") as f:
                    f.write(text)
    return files


if __name__ == "__main__":
    for p in generate():
        print("wrote", os.path.relpath(p, ROOT))
