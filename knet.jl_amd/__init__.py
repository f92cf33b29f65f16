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
from .loss import nll, findindices, accuracy, ungetindex, bce, logistic
from .indexing import (getcols, getrows, setcols_, setrows_, addcols_, addrows_, setents_, getindex2, setindex2_, icat, concat,
                       getindex, setindex_)
from .dropout import dropout, dropback, dropout_, dropback_
from .update import SGD, Momentum, Nesterov, Adagrad, Rmsprop, Adadelta, Adam, update_, gclip_
from .linalg import dense, matmul, mat, gemm, A_mul_B, A_mul_Bt, At_mul_B, axpy, scal, transpose, permutedims

libknet8()  # fail loudly at import time if the HIP library is missing
