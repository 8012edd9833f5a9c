"""Operators from the reference's examples and documentation, written against this package's DSL."""
from .accumulate import accumulate, cumsum, cumprod  # noqa: F401
from .expm1 import expm1, expm1_grad  # noqa: F401
from .log1p import log1p, log1p_grad  # noqa: F401
from .shift import shift_cyclic  # noqa: F401
from .elementwise import absolute  # noqa: F401
from .chain import chain8  # noqa: F401
from .indexed import gather_transpose  # noqa: F401
from .conv1d import conv_1d  # noqa: F401
from .graph import triangles_op, triangles, adjacency_from_edges  # noqa: F401
