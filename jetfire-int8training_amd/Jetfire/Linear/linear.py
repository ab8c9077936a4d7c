"""int8_linear_forward / int8_linear_backward on top of the BlockQuantizeCUDA extension.

Data format everywhere: codes int8 [..., R, C] with one scale per 32x32 tile, scales [..., R/32, C/32]
(float16 as in the reference, float32 accepted).  The GEMM entry points take their scale operands as [K/32, rows/32];
the reference makes transposed copies for that (linear_fwd.py:17-18, linear_bwd.py:11), here the .t() VIEW of the
block tensor's own scale array is passed and the kernel reads it in place.  The zero bias the reference allocates on
every call (linear_fwd.py:20-21) is kept per device and width.  The weight-gradient GEMM reads the gradient
[tokens, C_out] in place as its [K, M] operand when no pre-transposed copy is supplied (G8T=None); the reference needs
the copy (linear_bwd.py:21, made by int8_transpose / int8_quantize_transpose).

Bias (sketched in the reference, JetfireGEMMKernel/BlockQuantize/QBlockLinear.py:38-39, 63-66; its recipe runs without):
`bias=` of the forward functions is added to the accumulator in the kernel's requantising epilogue with
biasmax = max|bias| added to the block absmax (…BiasRowCol.cu:313,357); `bias_grad=True` of the backward functions
also returns the bias gradient, the column sums of the (dequantised) output gradient.

Every kernel is reached through the C++ extension (BlockQuantizeCUDA and its submodule BlockQuantizeCUDA.jetfire).
"""
import os
import sys

import torch

_PKG = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if _PKG not in sys.path:
    sys.path.insert(0, _PKG)

import BlockQuantizeCUDA as BQC  # noqa: E402

_jf = BQC.jetfire       # GEMMs with fused epilogues, column sums


def _flat2(t):
    """[..., C] -> [prod(...), C] without copying when possible."""
    return t.reshape(-1, t.shape[-1])


def _k_major(s2d):
    """[rows/32, K/32] -> [K/32, rows/32] without a copy (the extension accepts this view)."""
    return s2d.contiguous().t()


_ZERO_BIAS = {}


def _zero_bias(n, device):
    key = (str(device), n)
    if key not in _ZERO_BIAS:
        _ZERO_BIAS[key] = (torch.zeros(n, dtype=torch.float32, device=device), torch.zeros(1, dtype=torch.float32, device=device))
    return _ZERO_BIAS[key]


def bias_operands(bias, n_out, device):
    """(bias as contiguous float32 [N], biasmax = max|bias| as float32 [1]) for the kernel; the zero pair for None."""
    if bias is None:
        return _zero_bias(n_out, device)
    if bias.numel() != n_out:
        raise RuntimeError(f"bias must have {n_out} elements, got {bias.numel()}")
    b = bias.detach().reshape(-1).to(torch.float32).contiguous()
    return b, b.abs().max().reshape(1)


def _bias_pair(bias, n_out, device):
    """bias may already be the (bias, biasmax) pair (a caller that caches it per parameter version)."""
    if isinstance(bias, tuple):
        return bias
    return bias_operands(bias, n_out, device)


def _check_block(B):
    if B != 32:
        raise RuntimeError(f"the INT8 GEMM kernels use 32x32 quantisation blocks, got B={B}")


def int8_linear_forward(X8_3D, SX16_3D, W8, SW16, output_quantized, B, bias=None):
    """Y = X W^T (+ bias).  X8 [BS,T,K] (or [M,K]), SX [BS,T/32,K/32]; W8 [N,K], SW [N/32,K/32]; bias [N] or None.
    Returns (O8 [BS,T,N], SO [BS,T/32,N/32]) or, with output_quantized=False, the dequantised
    output in the scale dtype (reference: linear_fwd.py:4-32; bias: QBlockLinear.py:38-39)."""
    _check_block(B)
    lead = tuple(X8_3D.shape[:-1])
    s_lead = tuple(SX16_3D.shape[:-1])
    x2 = _flat2(X8_3D)
    sx2 = _flat2(SX16_3D)
    n_out = W8.shape[0]
    m, k = x2.shape
    b, bmax = _bias_pair(bias, n_out, W8.device)
    if not output_quantized:
        # the quantising GEMM and the codes x scales product of the reference (linear_fwd.py:22-31) in one kernel: same bits
        out = _jf.igemm_block_q_dequant(x2.contiguous(), W8.contiguous(), _k_major(sx2), _k_major(SW16), _jf.B_NK,
                                        SW16.dtype, b, bmax)
        return out.reshape(*lead, n_out)
    o8, so = BQC.igemm_output_int_quantize_bias_rowcol(x2.contiguous(), W8.t(), b, bmax,
                                                       _k_major(sx2), _k_major(SW16), m, n_out, k)
    return o8.reshape(*lead, n_out), so.reshape(*s_lead, SW16.shape[0])


def int8_linear_forward_gelu(X8_3D, SX16_3D, W8, SW16, B, approximate="none", bias=None):
    """int8_linear_forward(..., output_quantized=True) followed by int8_gelu_forward, in one kernel (no counterpart in
    the reference, whose MLP runs the two back to back, qmodel.py:210-214).  Returns (O8, SO, G8, SG): the linear
    output (kept for the backward pass) and its GELU (the next layer's input), bit-identical to the two separate calls."""
    _check_block(B)
    if approximate not in ("none", "tanh"):
        raise RuntimeError("approximate must be 'none' or 'tanh'")
    lead, s_lead = tuple(X8_3D.shape[:-1]), tuple(SX16_3D.shape[:-1])
    x2, sx2 = _flat2(X8_3D).contiguous(), _flat2(SX16_3D)
    n_out = W8.shape[0]
    b, bmax = _bias_pair(bias, n_out, W8.device)
    o8, so, g8, sg = _jf.igemm_block_q_gelu(x2, W8.contiguous(), _k_major(sx2), _k_major(SW16),
                                            _jf.GELU_TANH if approximate == "tanh" else _jf.GELU_ERF,
                                            0.0 if approximate == "tanh" else 5e-5,   # as Nonlinear.int8_gelu_forward
                                            b, bmax)
    shp, sshp = (*lead, n_out), (*s_lead, SW16.shape[0])
    return o8.reshape(shp), so.reshape(sshp), g8.reshape(shp), sg.reshape(sshp)


def int8_linear_backward(X8_3D, SX16_3D, G8_3D, SG16_3D, G8T, W8, SW16, B, stochastic=True, dgrad_quantize=True,
                         wgrad_splitk=1, wgrad_dtype=None, bias_grad=False):
    """dX = dY W (requantised with stochastic rounding) and dW = dY^T X (fp16).
    G8 [BS,T,N] with SG [BS,T/32,N/32]; G8T = G8 transposed to [N, BS*T], or None (then G8 itself is read, no copy);
    W8 [N,K], SW [N/32,K/32].
    Returns (GX8, GSX, GW) or (GX_fp, GW) when dgrad_quantize=False (reference: linear_bwd.py:4-29; like
    there, the activation gradient is always rounded stochastically).  wgrad_splitk (not in the reference): 1 = its
    arithmetic; 0 = let the library cut K into ordered partial sums when dW has too few tiles to fill the GPU.
    wgrad_dtype (not in the reference): None = float16 as there; float32 / bfloat16 = dW leaves the kernel in that type.
    bias_grad=True appends the bias gradient (float32 [N], the column sums of G8 x SG; QBlockLinear.py:63-66)."""
    _check_block(B)
    g2, sg2 = _flat2(G8_3D).contiguous(), _flat2(SG16_3D).contiguous()
    x2, sx2 = _flat2(X8_3D).contiguous(), _flat2(SX16_3D).contiguous()
    tokens, c_out = g2.shape
    c_in = W8.shape[1]
    gb = (_jf.block_colsum(g2, sg2),) if bias_grad else ()
    if dgrad_quantize:
        gx8, gsx = BQC.igemm_output_int_quantize_stochastic(g2, W8, _k_major(sg2), SW16, tokens, c_in, c_out)
    else:
        # the stochastic quantising GEMM and the codes x scales product of the reference (linear_bwd.py:17,26-28) in one
        # kernel: same bits, same noise counters
        gx = _jf.igemm_block_q_dequant(g2, W8.contiguous(), _k_major(sg2), SW16, _jf.B_KN, SW16.dtype, None, None,
                                       _jf.ROUND_STOCHASTIC)
    if G8T is None:
        G8T = g2.t()                                               # a view: the extension reads g2 as the [K, M] operand
    gw = BQC.igemm_output_fp_no_quantize(G8T, x2, sg2, sx2, G8T.shape[0], c_in, G8T.shape[1], wgrad_splitk, wgrad_dtype)
    if not dgrad_quantize:
        return (gx.reshape(*G8_3D.shape[:-1], c_in), gw) + gb
    return (gx8.reshape(*G8_3D.shape[:-1], c_in), gsx.reshape(*SG16_3D.shape[:-1], SW16.shape[1]), gw) + gb


def int8_linear_backward_gelu(X8_3D, SX16_3D, G8_3D, SG16_3D, W8, SW16, PRE8_3D, SPRE16_3D, B, approximate="none",
                              stochastic=True, wgrad_splitk=1, wgrad_dtype=None, bias_grad=False):
    """int8_linear_backward(...) followed by int8_gelu_backward(PRE8, SPRE, <its activation gradient>, ...), with the
    GELU backward running in the epilogue of the activation-gradient GEMM (no counterpart in the reference, whose MLP
    backward runs the two back to back, qmodel.py:249-253).  X8 / SX: the linear layer's input (= the GELU's output),
    PRE8 / SPRE: the GELU's input; G8 [BS,T,N], W8 [N,K].  Returns (GPRE8, GSPRE, GW): the gradient with respect to the
    GELU's input, requantised (`stochastic` as in int8_gelu_backward), and the weight gradient; bit-identical to the
    two separate calls (which draw their rounding noise in the same order)."""
    _check_block(B)
    if approximate not in ("none", "tanh"):
        raise RuntimeError("approximate must be 'none' or 'tanh'")
    g2, sg2 = _flat2(G8_3D).contiguous(), _flat2(SG16_3D).contiguous()
    x2, sx2 = _flat2(X8_3D).contiguous(), _flat2(SX16_3D).contiguous()
    p2, sp2 = _flat2(PRE8_3D).contiguous(), _flat2(SPRE16_3D).contiguous()
    tokens, c_out = g2.shape
    c_in = W8.shape[1]
    gp8, gsp = _jf.igemm_block_q_gelu_bwd(g2, W8.contiguous(), _k_major(sg2), SW16, p2, sp2,
                                          _jf.GELU_TANH if approximate == "tanh" else _jf.GELU_ERF,
                                          _jf.ROUND_STOCHASTIC if stochastic else _jf.ROUND_NEAREST)
    gw = BQC.igemm_output_fp_no_quantize(g2.t(), x2, sg2, sx2, c_out, c_in, tokens, wgrad_splitk, wgrad_dtype)
    gb = (_jf.block_colsum(g2, sg2),) if bias_grad else ()
    return (gp8.reshape(*G8_3D.shape[:-1], c_in), gsp.reshape(*SG16_3D.shape[:-1], SW16.shape[1]), gw) + gb
