"""Per-block INT8 linear layer, forward and backward (same names and signatures as the reference's
Jetfire/Linear package: linear_fwd.py:4, linear_bwd.py:4)."""
from .linear import int8_linear_backward, int8_linear_forward

__all__ = ["int8_linear_forward", "int8_linear_backward"]
