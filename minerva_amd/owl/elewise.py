"""Element-wise operators with the names and argument conventions of the reference's
owl/owl/elewise.py:6-87 (the gradient helpers take the forward output where cuDNN's
activation-backward takes both output and input)."""
from . import NArray


def mult(x, y):
    """Element-wise product (`x * y` is the matrix product)."""
    return NArray.mult(x, y)


def exp(x):
    return NArray.exp(x)


def ln(x):
    return NArray.ln(x)


def sigm(x):
    return NArray.sigm(x)


def relu(x):
    return NArray.relu(x)


def tanh(x):
    return NArray.tanh(x)


def sigm_back(y, x=None):
    """Gradient through a sigmoid: y is the incoming gradient, x the sigmoid's output.
    (The reference's one-argument form hands y on without the forward output,
    elewise.py:61-68, which its binding does not accept; both arguments are needed.)"""
    if x is None:
        raise TypeError("sigm_back needs the gradient and the forward output")
    return NArray.sigm_back(y, x, x)


def relu_back(y, x):
    """Gradient through a ReLU: y is the incoming gradient, x the ReLU's output
    (elewise.py:70-78)."""
    return NArray.relu_back(y, x, x)


def tanh_back(y, x=None):
    if x is None:
        raise TypeError("tanh_back needs the gradient and the forward output")
    return NArray.tanh_back(y, x, x)
