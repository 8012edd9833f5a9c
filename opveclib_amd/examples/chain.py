"""The element-wise chain of eight operators that the fusion optimizer turns into one kernel: add, mul by a scalar
tensor, tanh, sigmoid (stdops), log1p, expm1 (the reference's examples), sub (stdops) and the absolute value (the
reference's documentation example)."""

from .. import stdops
from .elementwise import absolute
from .expm1 import expm1
from .log1p import log1p


def chain8(a, b, s):
    """``|expm1(log1p(sigmoid(tanh((a + b) * s)))) - b|`` as eight operators; returns every stage's operator."""
    t1 = stdops.add(a, b)
    t2 = stdops.mul(t1, s)
    t3 = stdops.tanh(t2)
    t4 = stdops.sigmoid(t3)
    t5 = log1p(t4)
    t6 = expm1(t5)
    t7 = stdops.sub(t6, b)
    y = absolute(t7)
    return [t1, t2, t3, t4, t5, t6, t7, y]
