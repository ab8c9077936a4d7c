"""Per-block INT8 linear layer, forward and backward (same names and signatures as the reference's
Jetfire/Linear package: linear_fwd.py:4, linear_bwd.py:4), plus the forward with the GELU fused into its epilogue and
the backward with the GELU backward fused into the epilogue of its activation-gradient GEMM."""
from .linear import int8_linear_backward, int8_linear_backward_gelu, int8_linear_forward, int8_linear_forward_gelu

__all__ = ["int8_linear_forward", "int8_linear_backward", "int8_linear_forward_gelu", "int8_linear_backward_gelu"]
