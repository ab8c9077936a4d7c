"""Memory-bound operators of the INT8 data flow (same names and signatures as the reference's
Jetfire/Nonlinear package, __init__.py:1-8), each one a hand-written gfx950 kernel."""
from .common import SCALE_MIN_THRES
from .ops import (int8_add_Ifp_Ig16_Ofp_Og, int8_add_Ifp_Ig16_Ofp_Og_MeanVar, int8_column_sums, int8_dequantize, int8_gelu_backward,
                  int8_gelu_forward, int8_layernorm_backward, int8_layernorm_backward_add, int8_layernorm_forward, int8_quantize,
                  int8_quantize_concat, int8_quantize_transpose, int8_rowstats, int8_transpose)

__all__ = ["SCALE_MIN_THRES", "int8_quantize", "int8_quantize_transpose", "int8_transpose", "int8_dequantize",
           "int8_layernorm_forward", "int8_layernorm_backward", "int8_gelu_forward", "int8_gelu_backward",
           "int8_add_Ifp_Ig16_Ofp_Og", "int8_add_Ifp_Ig16_Ofp_Og_MeanVar", "int8_rowstats", "int8_quantize_concat",
           "int8_layernorm_backward_add", "int8_column_sums"]
