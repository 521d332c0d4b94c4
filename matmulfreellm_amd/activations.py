"""swiglu (interface of mmfreelm/modules/activations.py:178)."""
from . import functional as F_


def swiglu(x, y):
    """x * sigmoid(x) * y computed in fp32 as (x*y)/(1+exp(-x)), returned in x.dtype."""
    from .autograd import SwiGLUFn, needs_grad
    if needs_grad(x, y):
        return SwiGLUFn.apply(x, y)
    return F_.swiglu(x, y)
