"""Random block tensors for tests and benchmarks (counterpart of Jetfire/Nonlinear/utils.py:3-15)."""
import torch


def random_tensor_generator(BS, SL, CDIM, QB, dtype):
    """Returns (dequantised values, int8 codes [BS,SL,CDIM], scales [BS,SL/QB,CDIM/QB] float16)."""
    codes = torch.randn(BS, SL, CDIM, dtype=dtype, device="cuda")
    codes = (codes * 127 / codes.abs().max()).to(torch.int8)
    scales = torch.randn(BS, SL // QB, CDIM // QB, device="cuda").to(torch.float16)
    wide = scales.repeat_interleave(QB, dim=1).repeat_interleave(QB, dim=2)
    return codes.to(wide.dtype) * wide, codes, scales
