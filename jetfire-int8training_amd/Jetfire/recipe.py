"""INT8 data-flow transformer block built on the Linear / Nonlinear operators.

Counterpart of the autograd Functions of the reference recipe (INT8_GPT2/qmodel.py:86-171 attention,
:190-268 MLP, :295-363 model begin/end): between Functions an activation travels as the triple
(fp residual, INT8 codes, per-block scales [, row mean, row rstd]) and a gradient as (fp residual grad, INT8 codes,
scales).  Autograd only carries floating tensors, so the INT8 codes cross Function boundaries re-viewed as
float8_e4m3fn (same bytes), exactly as the reference does (qmodel.py:131,153,230,266).

Two per-call costs of the reference are gone: weights are quantised once per weight version (WeightCodes below), and no
transposed gradient is materialised for the weight-gradient GEMMs (the reference calls int8_transpose /
int8_quantize_transpose before every one, qmodel.py:156,237,250; here the GEMM reads the gradient in place).  Weight
gradients with too few output tiles to fill the GPU are computed with the library's K split (ordered fp32 partial sums).

Linear biases: the reference's recipe runs without them (its kernel has the inputs, qmodel.py never passes any);
here QBlock(..., bias=True) gives the four linear layers a bias that is added in the GEMM's requantising epilogue
(JetfireGEMMKernel/BlockQuantize/QBlockLinear.py:38-39) and whose gradient is the column sum of the layer's quantised
output gradient (:63-66).  LayerNorm has a weight only.
"""
import weakref

import torch
import torch.nn as nn
import torch.nn.functional as F

from Linear import int8_linear_backward, int8_linear_backward_gelu, int8_linear_forward, int8_linear_forward_gelu
from Linear.linear import bias_operands
from Nonlinear import (int8_add_Ifp_Ig16_Ofp_Og_MeanVar, int8_layernorm_backward_add, int8_layernorm_forward, int8_quantize,
                       int8_quantize_concat)

QB = 32
_F8 = torch.float8_e4m3fn


class WeightCodes:
    """INT8 codes and scales of weights, made once per weight VERSION instead of once per forward.

    The reference re-quantises every weight in every forward (qmodel.py:92,139,199-200) although a weight only changes
    in the optimizer step.  A tensor's version counter is bumped by every in-place update (optimizer steps, `copy_`,
    `add_` under no_grad), so (tensor identity, version) names the weight's current value; deterministic rounding makes
    the cached codes identical to re-quantised ones.  Entries die with their tensors."""

    def __init__(self):
        self._entries = {}
        self.hits = self.misses = 0

    def get(self, w):
        key = id(w)
        e = self._entries.get(key)
        if e is not None and e[0]() is w and e[1] == w._version and e[2] == w.data_ptr():
            self.hits += 1
            return e[3], e[4]
        self.misses += 1
        q, s = int8_quantize(w.detach(), QB)
        self._entries[key] = (weakref.ref(w, lambda _r, k=key, d=self._entries: d.pop(k, None)), w._version, w.data_ptr(), q, s)
        return q, s

    def get_bias(self, b):
        """(bias as float32, max|bias| as a one-element tensor) of a bias parameter, made once per version like the
        weight codes; None for None."""
        if b is None:
            return None
        key = id(b)
        e = self._entries.get(key)
        if e is not None and e[0]() is b and e[1] == b._version and e[2] == b.data_ptr():
            self.hits += 1
            return e[3], e[4]
        self.misses += 1
        b32, bmax = bias_operands(b, b.numel(), b.device)
        self._entries[key] = (weakref.ref(b, lambda _r, k=key, d=self._entries: d.pop(k, None)), b._version, b.data_ptr(), b32, bmax)
        return b32, bmax

    def clear(self):
        self._entries.clear()


weight_codes = WeightCodes()


def _as_f8(q):
    return q.view(_F8)


def _as_s8(q):
    return q.view(torch.int8)


class StreamBegin(torch.autograd.Function):
    """fp activation -> (fp, codes, scales).  Gradient: the fp gradient passes through (qmodel.py:309-327)."""

    @staticmethod
    def forward(ctx, x):
        q, s = int8_quantize(x, QB)
        return x, _as_f8(q), s

    @staticmethod
    def backward(ctx, g, _qg, _sg):
        return g


class StreamEnd(torch.autograd.Function):
    """(fp, codes, scales) -> fp.  Gradient: the fp gradient plus its stochastic block quantisation
    (qmodel.py:343-362)."""

    @staticmethod
    def forward(ctx, x, qx, sx):
        return x

    @staticmethod
    def backward(ctx, g):
        qg, sg = int8_quantize(g.contiguous(), QB, stochastic=True)
        return g, _as_f8(qg), sg


class AttentionIn(torch.autograd.Function):
    """LayerNorm -> QKV projection, fp16 out for the attention kernel (qmodel.py:86-131).  Q, K and V leave as three
    views of the projection's output, so that their gradients come back as three tensors and are quantised where they
    lie: the concatenated gradient the reference quantises (autograd's cat behind the split of qkv, 78 MB at GPT-2 XL
    size) is never made; codes, scales and rounding noise are those of the concatenation."""

    @staticmethod
    def forward(ctx, residual, qx, sx, w_qkv, ln_w, mean, rstd, b_qkv=None):
        qw, sw = weight_codes.get(w_qkv)
        ctx.wdtype = w_qkv.dtype          # the weight gradient leaves its GEMM in the parameter's type: no conversion kernel
        ctx.res_dtype = residual.dtype    # and the residual's gradient leaves the add in the residual's type
        ctx.bias_dtype = None if b_qkv is None else b_qkv.dtype
        qx = _as_s8(qx)
        qn, sn, _ = int8_layernorm_forward(qx, sx, ln_w, mean, rstd, QB)
        qkv = int8_linear_forward(qn, sn, qw, sw, False, QB, bias=weight_codes.get_bias(b_qkv))
        ctx.save_for_backward(qx, sx, qn, sn, qw, sw, ln_w, mean, rstd)
        q, k, v = qkv.split(qkv.shape[-1] // 3, dim=-1)
        return residual, q, k, v

    @staticmethod
    def backward(ctx, fpg, gq, gk, gv):
        qx, sx, qn, sn, qw, sw, ln_w, mean, rstd = ctx.saved_tensors
        qg, sg = int8_quantize_concat([gq, gk, gv], QB, stochastic=True)
        qg, sg, gw, *gb = int8_linear_backward(qn, sn, qg, sg, None, qw, sw, QB, stochastic=True, wgrad_splitk=0,
                                               wgrad_dtype=ctx.wdtype, bias_grad=ctx.bias_dtype is not None)
        # LayerNorm backward and the residual add behind it (qmodel.py:125-128) as one kernel, same bits
        res_g, qg, sg, g_ln = int8_layernorm_backward_add(qx, sx, qg, sg, ln_w, QB, mean, rstd, fpg.contiguous(), stochastic=True,
                                                          add_stochastic=True, out_dtype=ctx.res_dtype)
        return res_g, _as_f8(qg), sg, gw, g_ln, None, None, (gb[0].to(ctx.bias_dtype) if gb else None)


def _attention_out_forward(residual, y, w_proj, b_proj=None):
    """quantise -> output projection -> residual add with the next LayerNorm's statistics (qmodel.py:134-153); the sum is
    float32 as in the reference.  Returns the outputs and what the backward needs."""
    qw, sw = weight_codes.get(w_proj)
    qy, sy = int8_quantize(y.contiguous(), QB)
    qo, so = int8_linear_forward(qy, sy, qw, sw, True, QB, bias=weight_codes.get_bias(b_proj))
    fp, q, s, mean, rstd = int8_add_Ifp_Ig16_Ofp_Og_MeanVar(residual.contiguous(), qo, so, QB)
    return (fp, q, s, mean, rstd), (qy, sy, qw, sw)


def _attention_out_backward(saved, qg, sg, wdtype, bias_dtype=None):
    """gradient of the attention output (fp16 / bf16 for the attention kernel's backward), of the projection's
    weight (qmodel.py:155-171) and, with a bias, of the bias: (g, gw, gb or None)"""
    qy, sy, qw, sw = saved
    g, gw, *gb = int8_linear_backward(qy, sy, qg, sg, None, qw, sw, QB, stochastic=True, dgrad_quantize=False, wgrad_splitk=0,
                                      wgrad_dtype=wdtype, bias_grad=bias_dtype is not None)
    return g, gw, (gb[0].to(bias_dtype) if gb else None)


def _mlp_forward(residual, qx, sx, w_fc, w_proj, ln_w, mean, rstd, out_dtype, b_fc=None, b_proj=None):
    """LayerNorm -> fc + GELU -> proj -> residual add (qmodel.py:193-231).  out_dtype: type of the fp sum that leaves the
    block (the reference casts it to bfloat16, qmodel.py:228; here the add kernel writes it in that type)."""
    qw1, sw1 = weight_codes.get(w_fc)
    qw2, sw2 = weight_codes.get(w_proj)
    qn, sn, _ = int8_layernorm_forward(qx, sx, ln_w, mean, rstd, QB)
    qh, sh, qa, sa = int8_linear_forward_gelu(qn, sn, qw1, sw1, QB, bias=weight_codes.get_bias(b_fc))   # fc and its GELU in one kernel
    qo, so = int8_linear_forward(qa, sa, qw2, sw2, True, QB, bias=weight_codes.get_bias(b_proj))
    outs = int8_add_Ifp_Ig16_Ofp_Og_MeanVar(residual.contiguous(), qo, so, QB, out_dtype=out_dtype)
    return outs, (qx, sx, qn, sn, qh, sh, qa, sa, qw1, sw1, qw2, sw2, ln_w, mean, rstd)


def _mlp_backward(saved, fpg, qg, sg, wdtype, res_dtype, bias_dtype=None):
    """(qmodel.py:233-267); the residual's gradient leaves the add in res_dtype.  Returns (res_g, qg, sg, gw1, gw2, g_ln,
    gb1, gb2), the bias gradients None without biases."""
    qx, sx, qn, sn, qh, sh, qa, sa, qw1, sw1, qw2, sw2, ln_w, mean, rstd = saved
    want_gb = bias_dtype is not None
    # proj's backward with the GELU backward in the epilogue of its activation-gradient GEMM (one kernel for
    # int8_linear_backward's dgrad + int8_gelu_backward, same bits)
    qg, sg, gw2, *gb2 = int8_linear_backward_gelu(qa, sa, qg, sg, qw2, sw2, qh, sh, QB, stochastic=True, wgrad_splitk=0,
                                                  wgrad_dtype=wdtype, bias_grad=want_gb)
    qg, sg, gw1, *gb1 = int8_linear_backward(qn, sn, qg, sg, None, qw1, sw1, QB, stochastic=True, wgrad_splitk=0, wgrad_dtype=wdtype,
                                             bias_grad=want_gb)
    # LayerNorm backward and the residual add behind it (qmodel.py:258-261) as one kernel, same bits
    res_g, qg, sg, g_ln = int8_layernorm_backward_add(qx, sx, qg, sg, ln_w, QB, mean, rstd, fpg.contiguous(), stochastic=True,
                                                      add_stochastic=True, out_dtype=res_dtype)
    return (res_g, qg, sg, gw1, gw2, g_ln, (gb1[0].to(bias_dtype) if gb1 else None), (gb2[0].to(bias_dtype) if gb2 else None))


class AttentionOut(torch.autograd.Function):
    """Output projection + residual add, producing the statistics of the next LayerNorm (qmodel.py:134-171)."""

    @staticmethod
    def forward(ctx, residual, y, w_proj, b_proj=None):
        ctx.wdtype = w_proj.dtype
        ctx.bias_dtype = None if b_proj is None else b_proj.dtype
        ctx.set_materialize_grads(False)  # mean / rstd receive no gradient: None instead of two zero-filled tensors
        (fp, q, s, mean, rstd), saved = _attention_out_forward(residual, y, w_proj, b_proj)
        ctx.save_for_backward(*saved)
        return fp, _as_f8(q), s, mean, rstd

    @staticmethod
    def backward(ctx, fpg, qg, sg, _m, _r):
        g, gw, gb = _attention_out_backward(ctx.saved_tensors, _as_s8(qg), sg, ctx.wdtype, ctx.bias_dtype)
        return fpg, g, gw, gb


class MLPResidual(torch.autograd.Function):
    """LayerNorm -> fc -> GELU -> proj -> residual add, all on INT8 block tensors (qmodel.py:190-268)."""

    @staticmethod
    def forward(ctx, residual, qx, sx, w_fc, w_proj, ln_w, mean, rstd, out_dtype=torch.float32, b_fc=None, b_proj=None):
        ctx.wdtype = w_fc.dtype
        ctx.res_dtype = residual.dtype
        ctx.bias_dtype = None if b_fc is None else b_fc.dtype
        ctx.set_materialize_grads(False)  # as in AttentionOut
        (fp, q, s, mean2, rstd2), saved = _mlp_forward(residual, _as_s8(qx), sx, w_fc, w_proj, ln_w, mean, rstd, out_dtype, b_fc, b_proj)
        ctx.save_for_backward(*saved)
        return fp, _as_f8(q), s, mean2, rstd2

    @staticmethod
    def backward(ctx, fpg, qg, sg, _m, _r):
        res_g, qg, sg, gw1, gw2, g_ln, gb1, gb2 = _mlp_backward(ctx.saved_tensors, fpg, _as_s8(qg), sg, ctx.wdtype, ctx.res_dtype,
                                                                ctx.bias_dtype)
        return res_g, _as_f8(qg), sg, gw1, gw2, g_ln, None, None, None, gb1, gb2


class AttentionOutMLP(torch.autograd.Function):
    """AttentionOut followed by MLPResidual as ONE autograd node, same kernels and same bits.  The float32 sum between
    the two halves and its gradient then never cross an autograd edge, so the gradient can leave its add kernel in the
    type of the residual that receives it: with a bfloat16 stream between blocks (qmodel.py:228) the reference's
    float32 gradient of that sum is cast by autograd when it reaches the bfloat16 residual, a pass of its own."""

    @staticmethod
    def forward(ctx, residual, y, w_attn_proj, w_fc, w_mlp_proj, ln_w, out_dtype, b_attn_proj=None, b_fc=None, b_mlp_proj=None):
        ctx.wdtype = w_fc.dtype
        ctx.res_dtype = residual.dtype
        ctx.bias_dtype = None if b_fc is None else b_fc.dtype
        ctx.set_materialize_grads(False)
        (mid, q, s, mean, rstd), saved_a = _attention_out_forward(residual, y, w_attn_proj, b_attn_proj)
        (fp, q, s, mean2, rstd2), saved_m = _mlp_forward(mid, q, s, w_fc, w_mlp_proj, ln_w, mean, rstd, out_dtype, b_fc, b_mlp_proj)
        ctx.n_a = len(saved_a)
        ctx.save_for_backward(*saved_a, *saved_m)
        return fp, _as_f8(q), s, mean2, rstd2

    @staticmethod
    def backward(ctx, fpg, qg, sg, _m, _r):
        saved = ctx.saved_tensors
        res_g, qg, sg, gw1, gw2, g_ln, gb1, gb2 = _mlp_backward(saved[ctx.n_a:], fpg, _as_s8(qg), sg, ctx.wdtype, ctx.res_dtype,
                                                                ctx.bias_dtype)
        g, gwp, gbp = _attention_out_backward(saved[:ctx.n_a], qg, sg, ctx.wdtype, ctx.bias_dtype)
        return res_g, g, gwp, gw1, gw2, g_ln, None, gbp, gb1, gb2


class QBlock(nn.Module):
    """One pre-LayerNorm transformer block (causal self-attention + MLP) on the INT8 data flow.  out_dtype: type of the
    fp residual that leaves the block (float32, or the reference's bfloat16, qmodel.py:228).  bias=True: the four
    linear layers carry a bias (GPT-2's own configuration, qmodel.py:292), zero-initialised."""

    def __init__(self, n_embd, n_head, out_dtype=torch.float32, bias=False):
        super().__init__()
        assert n_embd % n_head == 0 and n_embd % QB == 0
        self.n_embd, self.n_head, self.out_dtype = n_embd, n_head, out_dtype
        mk = (lambda n: nn.Parameter(torch.zeros(n))) if bias else (lambda n: None)
        self.b_qkv, self.b_attn_proj, self.b_fc, self.b_mlp_proj = mk(3 * n_embd), mk(n_embd), mk(4 * n_embd), mk(n_embd)
        self.ln_1 = nn.Parameter(torch.ones(n_embd))
        self.ln_2 = nn.Parameter(torch.ones(n_embd))
        self.w_qkv = nn.Parameter(torch.randn(3 * n_embd, n_embd) * 0.02)
        self.w_attn_proj = nn.Parameter(torch.randn(n_embd, n_embd) * 0.02)
        self.w_fc = nn.Parameter(torch.randn(4 * n_embd, n_embd) * 0.02)
        self.w_mlp_proj = nn.Parameter(torch.randn(n_embd, 4 * n_embd) * 0.02)

    def forward(self, x, qx, sx, mean, rstd):
        B, T, C = x.shape
        res, q, k, v = AttentionIn.apply(x, qx, sx, self.w_qkv, self.ln_1, mean, rstd, self.b_qkv)
        q, k, v = (t.view(B, T, self.n_head, C // self.n_head).transpose(1, 2) for t in (q, k, v))
        y = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).contiguous().view(B, T, C)
        return AttentionOutMLP.apply(res, y, self.w_attn_proj, self.w_fc, self.w_mlp_proj, self.ln_2, self.out_dtype,
                                     self.b_attn_proj, self.b_fc, self.b_mlp_proj)


class QStack(nn.Module):
    """A stack of QBlocks between StreamBegin and StreamEnd: fp in, fp out (qmodel.py:418-446 without the
    embedding and the language-model head).  stream_dtype: type of the fp residual between blocks and of the output
    (the reference: bfloat16, qmodel.py:228); the input keeps its own type."""

    def __init__(self, n_layer, n_embd, n_head, stream_dtype=torch.float32, bias=False):
        super().__init__()
        self.blocks = nn.ModuleList(QBlock(n_embd, n_head, stream_dtype, bias) for _ in range(n_layer))

    def forward(self, x):
        x, qx, sx = StreamBegin.apply(x)
        mean = x.float().mean(dim=-1)
        rstd = torch.rsqrt(x.float().var(dim=-1, unbiased=False))
        for blk in self.blocks:
            x, qx, sx, mean, rstd = blk(x, qx, sx, mean, rstd)
        return StreamEnd.apply(x, qx, sx)
