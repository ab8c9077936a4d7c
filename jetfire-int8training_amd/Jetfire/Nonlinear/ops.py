"""The Nonlinear operators: shape handling over the C++ extension (BlockQuantizeCUDA.jetfire, csrc/jf_ops_ext.cpp), which
validates the tensors, allocates the outputs and enqueues the gfx950 kernels through the C ABI with the GIL released.

All functions accept 2-D [M,N] or 3-D [BS,T,N] operands like the reference launchers and return tensors
of matching rank; scales are float16 [.., M/32, N/32] unless the inputs carry float32 scales.
Stochastic rounding draws its Philox (seed, offset) from the device's default torch generator, so it follows
torch.manual_seed (the reference materialises a uniform_(-0.5,0.5) noise tensor, quantize.py:143-146).
"""
import os
import sys

import torch

_PKG = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if _PKG not in sys.path:
    sys.path.insert(0, _PKG)

import BlockQuantizeCUDA as _BQC  # noqa: E402

_jf = _BQC.jetfire      # the operators below, as C++ functions on 2-D tensors

from .common import SCALE_MIN_THRES  # noqa: E402


def _check_qb(QB):
    if QB != 32:
        raise RuntimeError(f"quantisation block size must be 32, got {QB}")


class _Shape:
    """Remembers how to fold 2-D results back to the rank of the input."""

    def __init__(self, t):
        if t.dim() not in (2, 3):
            raise RuntimeError(f"expected a 2-D or 3-D tensor, got {t.dim()} dimensions")
        self.batched = t.dim() == 3
        self.bs = t.shape[0] if self.batched else None

    def flat(self, t):
        return t.reshape(-1, t.shape[-1]).contiguous() if t is not None else None

    def fold(self, t):
        return t.reshape(self.bs, -1, t.shape[-1]) if self.batched else t

    def fold_vec(self, v):
        return v.reshape(self.bs, -1) if self.batched else v


def _f32(v):
    return v.reshape(-1).to(torch.float32).contiguous()


def int8_quantize(x, QB, stochastic=False, scale_dtype=torch.float16):
    """x fp32/fp16/bf16 -> (int8 codes, scales).  Reference: quantize.py:128-164."""
    _check_qb(QB)
    sh = _Shape(x)
    q, s, _ = _jf.quantize(sh.flat(x), _jf.ROUND_STOCHASTIC if stochastic else _jf.ROUND_NEAREST, scale_dtype)
    return sh.fold(q), sh.fold(s)


def int8_quantize_concat(xs, QB, stochastic=False, scale_dtype=torch.float16):
    """int8_quantize(torch.cat(xs, dim=-1), ...) without the concatenation (no counterpart in the reference, which
    quantises the concatenated gradient of the attention kernel's inputs, qmodel.py:112-120): every tensor of xs is
    quantised where it lies into its columns of the result.  Same codes, scales and noise as the two-step form."""
    _check_qb(QB)
    sh = _Shape(xs[0])
    flat = []
    for x in xs:
        if x.dim() != xs[0].dim() or x.shape[:-1] != xs[0].shape[:-1]:
            raise RuntimeError("tensors to concatenate must agree in all but the last dimension")
        f = x.reshape(-1, x.shape[-1])                             # a view whenever the leading dimensions can be merged
        in_place = (f.stride(1) == 1 and f.stride(0) >= f.shape[1]     # (an expanded gradient has row stride 0: copied)
                    and (f.stride(0) * f.element_size()) % 16 == 0 and f.data_ptr() % 16 == 0)
        flat.append(f if in_place else f.contiguous())
    q, s = _jf.quantize_slabs(flat, _jf.ROUND_STOCHASTIC if stochastic else _jf.ROUND_NEAREST, scale_dtype)
    return sh.fold(q), sh.fold(s)


def int8_quantize_transpose(x, QB, stochastic=False, transpose_output_2d=False, scale_dtype=torch.float16):
    """As int8_quantize, plus the transposed codes [N, M].  Reference: quantize_transpose.py:131-171."""
    _check_qb(QB)
    sh = _Shape(x)
    q, s, qt = _jf.quantize(sh.flat(x), _jf.ROUND_STOCHASTIC if stochastic else _jf.ROUND_NEAREST, scale_dtype, True)
    if sh.batched and not transpose_output_2d:
        qt = qt.reshape(sh.bs, -1, qt.shape[-1])
    return sh.fold(q), sh.fold(s), qt


def int8_transpose(x, transpose_output_2d=False):
    """int8 [M,N] -> [N,M] (3-D input is flattened over its leading dimensions first).  Reference: transpose.py:69-97."""
    sh = _Shape(x)
    y = _jf.transpose_s8(sh.flat(x))
    if sh.batched and not transpose_output_2d:
        y = y.reshape(sh.bs, -1, y.shape[-1])
    return y


def int8_dequantize(x, s_x, QB):
    """(codes, scales) -> float32.  Reference: dequantize.py:86-116."""
    _check_qb(QB)
    sh = _Shape(x)
    return sh.fold(_jf.dequantize(sh.flat(x), sh.flat(s_x), torch.float32))


def int8_rowstats(x, s_x, QB, eps=1e-5):
    """Per-row (mean, rstd) of a block tensor: the statistics int8_layernorm_forward consumes."""
    _check_qb(QB)
    sh = _Shape(x)
    mean, rstd = _jf.rowstats(sh.flat(x), sh.flat(s_x), eps)
    return sh.fold_vec(mean), sh.fold_vec(rstd)


def int8_layernorm_forward(x, sx, weight, mean, rstd, QB, eps=1e-6, bias=None):
    """dequant -> (x-mean)*rstd*weight (+bias) -> requant; returns (y, sy, (mean, rstd)).
    mean/rstd are per-row inputs as in the reference (layernorm.py:430-465, where `eps` is unused too);
    pass mean=None to have them computed from (x, sx) with this eps."""
    _check_qb(QB)
    sh = _Shape(x)
    x2, sx2 = sh.flat(x), sh.flat(sx)
    if mean is None or rstd is None:
        m2, r2 = _jf.rowstats(x2, sx2, eps)
        mean, rstd = sh.fold_vec(m2), sh.fold_vec(r2)
    qy, sy = _jf.layernorm_fwd(x2, sx2, _f32(weight), None if bias is None else _f32(bias), _f32(mean), _f32(rstd))
    return sh.fold(qy), sh.fold(sy), (mean, rstd)


def int8_layernorm_backward(x, sx, g, sg, w, QB, m, v, stochastic=False, eps=1e-6, return_dbias=False):
    """Returns (dx codes, dx scales, dweight[, dbias]).  m, v are the forward's (mean, rstd).
    Row reductions run over the full row (the reference reduces over its 128-column tile only,
    layernorm.py:331-332).  Reference launcher: layernorm.py:467-526."""
    _check_qb(QB)
    sh = _Shape(x)
    rounding = _jf.ROUND_STOCHASTIC if stochastic else _jf.ROUND_NEAREST
    qdx, sdx, dg, db = _jf.layernorm_bwd(sh.flat(x), sh.flat(sx), sh.flat(g), sh.flat(sg), _f32(w), _f32(m), _f32(v),
                                         rounding, want_dbeta=return_dbias)
    out = (sh.fold(qdx), sh.fold(sdx), dg.to(w.dtype))
    return out + (db.to(w.dtype),) if return_dbias else out


def int8_layernorm_backward_add(x, sx, g, sg, w, QB, m, v, x1, stochastic=False, add_stochastic=False, add_rounding="trunc",
                                out_dtype=torch.float32, return_dbias=False):
    """int8_layernorm_backward followed by int8_add_Ifp_Ig16_Ofp_Og(x1, dx, s_dx, ...) (the pair the reference's recipe
    calls back to back, qmodel.py:125-128, 258-261) as one kernel for rows of up to 2048 columns, same bits.
    Returns (y1, y2, s_y2, dweight[, dbias])."""
    _check_qb(QB)
    sh = _Shape(x)
    rounding = _jf.ROUND_STOCHASTIC if stochastic else _jf.ROUND_NEAREST
    y1, q, s, dg, db = _jf.layernorm_bwd_add(sh.flat(x), sh.flat(sx), sh.flat(g), sh.flat(sg), _f32(w), _f32(m), _f32(v),
                                             sh.flat(x1), rounding, _add_rounding(add_stochastic, add_rounding),
                                             want_dbeta=return_dbias, out_dtype=out_dtype)
    out = (sh.fold(y1), sh.fold(q), sh.fold(s), dg.to(w.dtype))
    return out + (db.to(w.dtype),) if return_dbias else out


def int8_gelu_forward(x, s_x, QB, approximate="none"):
    """dequant -> GELU -> requant.  'none' = erf form with SCALE_MIN_THRES added to the block absmax
    (reference: gelu_fwd.py:81,90); 'tanh' = tanh approximation, no threshold."""
    _check_qb(QB)
    sh = _Shape(x)
    if approximate == "none":
        qy, sy = _jf.gelu_fwd(sh.flat(x), sh.flat(s_x), _jf.GELU_ERF, SCALE_MIN_THRES)
    elif approximate == "tanh":
        qy, sy = _jf.gelu_fwd(sh.flat(x), sh.flat(s_x), _jf.GELU_TANH, 0.0)
    else:
        raise RuntimeError("approximate must be 'none' or 'tanh'")
    return sh.fold(qy), sh.fold(sy)


def int8_gelu_backward(x, s_x, g, s_g, QB, stochastic=False, approximate="none"):
    """(x, g) -> gelu'(x) * g, requantised.  Reference: gelu_bwd.py:173-215."""
    _check_qb(QB)
    sh = _Shape(x)
    if approximate not in ("none", "tanh"):
        raise RuntimeError("approximate must be 'none' or 'tanh'")
    qy, sy = _jf.gelu_bwd(sh.flat(x), sh.flat(s_x), sh.flat(g), sh.flat(s_g),
                          _jf.GELU_ERF if approximate == "none" else _jf.GELU_TANH,
                          _jf.ROUND_STOCHASTIC if stochastic else _jf.ROUND_NEAREST)
    return sh.fold(qy), sh.fold(sy)


def _add_rounding(stochastic, rounding):
    if rounding == "trunc":       # what the reference computes: .to(int8) without llrint (add.py:139)
        return _jf.ROUND_STOCHASTIC_TRUNC if stochastic else _jf.ROUND_TRUNC
    if rounding == "nearest":
        return _jf.ROUND_STOCHASTIC if stochastic else _jf.ROUND_NEAREST
    raise RuntimeError("rounding must be 'trunc' or 'nearest'")


def int8_add_Ifp_Ig16_Ofp_Og(x1, x2, s_x2, QB, stochastic=False, rounding="trunc", out_dtype=torch.float32):
    """y1 = x1 + dequant(x2) as float32, and its block quantisation (y2, s_y2).  Reference: add.py:164-211.
    out_dtype = float16 / bfloat16: y1 leaves the kernel already cast (what the reference's recipe does with a separate
    `.to()`, qmodel.py:228); y2, s_y2 are those of the fp32 sum either way."""
    _check_qb(QB)
    sh = _Shape(x1)
    y1, q, s, _, _ = _jf.add(sh.flat(x1), sh.flat(x2), sh.flat(s_x2), _add_rounding(stochastic, rounding), False, out_dtype)
    return sh.fold(y1), sh.fold(q), sh.fold(s)


def int8_add_Ifp_Ig16_Ofp_Og_MeanVar(x1, x2, s_x2, QB, rounding="trunc", out_dtype=torch.float32):
    """As above plus per-row (mean, rstd) of the fp32 y1 for the next LayerNorm: var = E[y^2] - mean^2,
    rstd = 1/sqrt(var), no epsilon (reference: add_mean_var.py:179-230, finishing step :219-221)."""
    _check_qb(QB)
    sh = _Shape(x1)
    # the statistics are finished by a second kernel inside the same call (the reference: eight torch operators)
    y1, q, s, mean, rstd = _jf.add(sh.flat(x1), sh.flat(x2), sh.flat(s_x2), _add_rounding(False, rounding), True, out_dtype)
    return sh.fold(y1), sh.fold(q), sh.fold(s), sh.fold_vec(mean), sh.fold_vec(rstd)


def int8_column_sums(g, s_g, QB):
    """Column sums over all rows of the block tensor (g, s_g), float32 [N]: the bias gradient of a linear layer from its
    quantised output gradient (sketched in the reference as G8.sum(0), QBlockLinear.py:63-66).  3-D operands are summed
    over both leading dimensions."""
    _check_qb(QB)
    sh = _Shape(g)
    return _jf.block_colsum(sh.flat(g), sh.flat(s_g))
