"""Standard element-wise operators with broadcasting and gradients (reference: opveclib/stdops)."""
from .math import *  # noqa: F401,F403
