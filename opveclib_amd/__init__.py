# Derived from opveclib/__init__.py of opveclib (https://github.com/opveclib/opveclib),
# Copyright 2016 Hewlett Packard Enterprise Development LP, licensed under the Apache License, Version 2.0
# (http://www.apache.org/licenses/LICENSE-2.0); see the NOTICE file at the root of this repository.
# Changes: the list of exported names is that project's; the names added here (set_math_mode, as_torch, CapturedDag, ...) are not.
"""
OVL for MI355X: the Operator Vectorization Library's DSL and operator API with a HIP (gfx950) backend.

The public names mirror the reference's opveclib/__init__.py:11-48.  ``as_tensorflow`` has no counterpart here;
``hip_enabled`` replaces ``cuda_enabled`` (which is kept as an alias).
"""

# @ Data types
from .expression import DType
from .expression import float16, float32, float64
from .expression import int8, int16, int32, int64
from .expression import uint8, uint16, uint32, uint64
from .expression import TensorType

# @ Expressions
from .expression import Scalar, Variable, InputTensor, OutputTensor, PositionTensor, LocalTensor

# @ Tensor functions
from .expression import position_in
from .expression import output, output_like
from .expression import zeros, ones

# @ Scalar functions
# @@ Utility
from .expression import variable, cast
# @@ Numeric limits
from .expression import min_value, max_value, epsilon
# @@ Unary math
from .expression import arccos, arcsin, arctan, cos, cosh, sin, sinh, tan, tanh
from .expression import exp, log, log10, sqrt
from .expression import ceil, absolute, floor
from .expression import logical_not
from .expression import isinf, isfinite, isnan
# @@ Binary math
from .expression import minimum, maximum, power, arctan2, logical_and, logical_or

# @ Control flow
from .expression import arange
from .expression import if_, elif_, else_

# @ Operator functions
from .operator import operator, gradient, evaluate, profile, set_math_mode, get_math_mode, set_trace_cache
from .autograd import as_torch
from .graph import CapturedDag

# @ Local runtime environment functions
from .local import version, logger, cache_directory, clear_op_cache
from . import local as _local


def __getattr__(name):
    if name in ('hip_enabled', 'cuda_enabled'):
        return getattr(_local, name)
    raise AttributeError('module %r has no attribute %r' % (__name__, name))
