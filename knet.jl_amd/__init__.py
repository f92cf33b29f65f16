"""Host-side mirror of the part of Knet.jl that sits on the backward-pass gradient path, backed by the
hand-written gfx950 kernels of ``libknet8.so``.

Names, argument order, 1-based ``dims``/labels and error behaviour follow the reference's Julia API
(``KnetArray``, ``relu``/``reluback``, ``sum(x; dims)``, ``logsoftmax``, ``nll``, ``dropout``, ``@diff``/``grad``/
``value`` as ``diff``/``grad``/``value``).  Importing the package loads the library; there is no CPU fallback.
"""
from .libknet8 import libknet8, knet8, LIB_PATH
from .karray import KnetArray, KnetPtr, Array, synchronize, Graph, capture
from .autograd import Param, diff, grad, value, recording
from .activation import (bias_act, relu, sigm, tanh, elu, selu, reluback, sigmback, tanhback, eluback, seluback,
                         gelu, hardsigmoid, hardswish, swish, tanh_, geluback, hardsigmoidback, hardswishback,
                         swishback, tanh_back, eluback21, seluback21, sigmback21, relu_kw, relu_kw_back,
                         unary_op, unary_op_with_degree, back11_op, back111_op)
from .reduction import sum, prod, maximum, minimum, sumabs, sumabs2, maxabs, minabs, countnz, reduce_op
from .binary import add, sub, mul, div, fill, zero, unbroadcast, broadcast_op
from .softmax import logsoftmax, softmax, logp, logsumexp, logsoftmaxback, softmaxback
from .cat import cat, hcat, vcat
from .statistics import mean, var, std, varm, stdm, norm, isequal, isapprox
from .random import seed_, rand_, randn_, RngState
from .loss import nll, findindices, accuracy, zeroone, ungetindex, bce, logistic
from .indexing import (getcols, getrows, setcols_, setrows_, addcols_, addrows_, setents_, getindex2, setindex2_, icat, concat,
                       getindex, setindex_)
from .dropout import dropout, dropback, dropout_, dropback_
from .update import SGD, Momentum, Nesterov, Adagrad, Rmsprop, Adadelta, Adam, update_, gclip_
from .train import (Data, minibatch, param, param0, params, gaussian, xavier, xavier_uniform, xavier_normal, Minimize, minimize, minimize_,
                    sgd, sgd_, momentum, momentum_, nesterov, nesterov_, adagrad, adagrad_, rmsprop, rmsprop_, adadelta, adadelta_,
                    adam, adam_, converge, converge_, train_, updates, epochs)
from .linalg import dense, dense_nll, matmul, mat, bmm, bmm_, gemm, A_mul_B, A_mul_Bt, At_mul_B, axpy, scal, transpose, permutedims

libknet8()  # fail loudly at import time if the HIP library is missing


# ---- operator sugar: a + b, a - b, a * b (elementwise, Julia's .*), a / b, -a, a @ b (matrix product, Julia's *) on KnetArray,
# Param and tape nodes; each is the primitive of the same name, so expressions written with operators are differentiable.
def _attach_operators():
    from . import autograd as _ag

    def _neg(a):
        return mul(a, -1)
    ops = {
        "__add__": lambda a, b: add(a, b), "__radd__": lambda a, b: add(b, a),
        "__sub__": lambda a, b: sub(a, b), "__rsub__": lambda a, b: sub(b, a),
        "__mul__": lambda a, b: mul(a, b), "__rmul__": lambda a, b: mul(b, a),
        "__truediv__": lambda a, b: div(a, b), "__rtruediv__": lambda a, b: div(b, a),
        "__matmul__": lambda a, b: matmul(a, b), "__rmatmul__": lambda a, b: matmul(b, a),
        "__neg__": _neg,
    }
    for cls in (KnetArray, _ag.Node, Param):
        for name, fn in ops.items():
            setattr(cls, name, fn)


from .binary import div  # noqa: E402
_attach_operators()
