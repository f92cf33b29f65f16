"""A small tape that plays AutoGrad.jl's part on the path this package covers.

AutoGrad.jl (1.2.4, a third-party dependency of the reference that is not part of its repository)
records primitives called on ``Param``s inside ``@diff`` and sweeps the tape backwards, calling the
gradient expression each ``@primitive`` declares and accumulating with ``addto!``.  This module
restates that published behaviour for the primitives on the gradient path:

    J = diff(lambda: nll(predict(w, x), y))      # @diff nll(predict(w,x),y)
    grad(J, w[0]); value(J)

Only what the MLP backward step needs is here: one level of recording (no nested ``diff``; the gradient functions
``reluback`` ... ``softmaxback`` are primitives with the reference's rules, so they can be differentiated when called directly), no Sparse containers.
"""
import numpy as np

from .karray import KnetArray

_TAPE = None  # the tape being recorded, or None outside diff()


def recording():
    """``AutoGrad.recording()`` -- what the reference's ``training()`` returns (src/Knet.jl:15)."""
    return _TAPE is not None


class Param:
    """A differentiable leaf (``Param(x)``, src/train20/param.jl:42-44)."""

    def __init__(self, value):
        self.value = value
        self.opt = None   # the optimizer `minimize` attaches (src/train20/train.jl:23-25); set beforehand to override it

    def __repr__(self):
        return "P(%r)" % (self.value,)


class Node:
    __slots__ = ("value", "parents", "back", "outgrad", "param")

    def __init__(self, value, parents=(), back=None, param=None):
        self.value, self.parents, self.back, self.outgrad, self.param = value, parents, back, None, param


class Tape:
    def __init__(self):
        self.nodes = []
        self.leaves = {}

    def leaf(self, p):
        n = self.leaves.get(id(p))
        if n is None:
            n = Node(p.value, param=p)
            self.leaves[id(p)] = n
            self.nodes.append(n)
        return n


def track(x):
    """Node of ``x`` on the current tape, or None if ``x`` does not depend on a Param."""
    if isinstance(x, Node):
        return x
    if isinstance(x, Param) and _TAPE is not None:
        return _TAPE.leaf(x)
    return None


def value(x):
    if isinstance(x, (Node, Param, Result)):
        return x.value
    return x


def primitive(fwd):
    """Decorator.  ``fwd(*values, **kw)`` returns ``(y, back)`` where ``back(dy)`` returns one gradient (or
    None) per positional argument; the wrapper records a node when any argument is tracked."""

    def wrapper(*args, **kw):
        nodes = [track(a) for a in args]
        vals = [value(a) for a in args]
        if _TAPE is None or all(n is None for n in nodes):
            out = fwd(*vals, **kw)
            return out[0]
        y, back = fwd(*vals, **kw)
        node = Node(y, tuple(nodes), back)
        _TAPE.nodes.append(node)
        return node

    wrapper.__name__ = getattr(fwd, "__name__", "primitive")
    wrapper.__doc__ = fwd.__doc__
    return wrapper


def selective(back):
    """Marks a gradient function ``back(dy, need)`` that computes only the gradients whose ``need`` entry is true."""
    back.selective = True
    return back


def addto(a, b):
    """``addto!(a,b)``: accumulate a gradient (src/autograd_gpu/addto.jl:7-10: ``axpy!(1,b,a)``)."""
    if a is None:
        return b
    if isinstance(a, KnetArray):
        # out of place: `a` may be shared with another node's gradient (identity rules pass dy through)
        from .binary import broadcast_op
        return broadcast_op("add", a, b)
    return a + b


class Result:
    """What ``@diff`` returns: the value plus the gradients of every Param that took part."""

    def __init__(self, value, grads, params=()):
        self.value, self.grads, self.params = value, grads, tuple(params)   # params: in order of first use (AutoGrad's params(J))


def diff(f):
    global _TAPE
    if _TAPE is not None:
        raise RuntimeError("nested diff() is not supported")
    tape = _TAPE = Tape()
    try:
        out = f()
    finally:
        _TAPE = None
    if not isinstance(out, Node):
        return Result(value(out), {})
    v = out.value
    if isinstance(v, KnetArray):
        if v.length != 1:
            raise ValueError("diff() needs a scalar result")
        out.outgrad = 1.0  # a scalar kept on the device (1-element array): see nll(..., fused=True) with device labels
    else:
        out.outgrad = type(v)(1) if isinstance(v, (np.floating, float)) else 1.0
    for node in reversed(tape.nodes):
        if node.outgrad is None or node.back is None:
            continue
        if getattr(node.back, "selective", False):
            # like AutoGrad, which evaluates a primitive's gradient expression only for the arguments that are tracked:
            # the input layer's product never computes the gradient wrt the data, a constant operand of .* is not summed
            grads = node.back(node.outgrad, tuple(p is not None for p in node.parents))
        else:
            grads = node.back(node.outgrad)
        for parent, g in zip(node.parents, grads):
            if parent is not None and g is not None:
                parent.outgrad = addto(parent.outgrad, g)
        if node.param is None:
            # Dead from here on: drop the gradient, the value and the closure that holds the saved activations, so their
            # device blocks go back to the pool while the sweep is still running -- what the reference's tape-aware
            # gcnode does after every node (src/autograd_gpu/gcnode.jl:63-93).
            node.outgrad = None
            node.back = None
            if node is not out:
                node.value = None
    return Result(v, {pid: n.outgrad for pid, n in tape.leaves.items()}, [n.param for n in tape.leaves.values()])


def grad(result, param):
    """``grad(J, w)``: gradient of the recorded scalar wrt ``param`` (None if it did not take part)."""
    return result.grads.get(id(param))
