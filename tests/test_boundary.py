"""The drop-in boundary: module BlockQuantizeCUDA and packages Linear / Nonlinear, imported the way
INT8_GPT2/qmodel.py:18-22 imports them, with the reference's names, argument order and return shapes."""
import inspect

import numpy as np
import pytest
import torch

from helpers import QB, rand_codes, rand_scales


# ------------------------------------------------------------------------------------------- CPU side
def test_imports_and_names():
    import BlockQuantizeCUDA as BQC
    from Linear import int8_linear_backward, int8_linear_forward  # noqa: F401
    from Nonlinear import (int8_add_Ifp_Ig16_Ofp_Og, int8_add_Ifp_Ig16_Ofp_Og_MeanVar, int8_gelu_backward,  # noqa: F401
                           int8_gelu_forward, int8_layernorm_backward, int8_layernorm_forward, int8_quantize,
                           int8_quantize_transpose, int8_transpose)
    for name in ("igemm_output_int_quantize_stochastic", "igemm_output_int_quantize_bias_rowcol",
                 "igemm_output_int_quantize_bias_rowrow", "igemm_output_int_quantize",
                 "igemm_output_int_quantize_fused", "igemm_output_fp_no_quantize", "igemm_basic_int8_gemm", "hgemm_v1"):
        assert callable(getattr(BQC, name)), name


# positional parameters of the reference launchers (Jetfire/Linear/*.py, Jetfire/Nonlinear/*.py)
SIGNATURES = {
    "Linear.int8_linear_forward": ["X8_3D", "SX16_3D", "W8", "SW16", "output_quantized", "B"],
    "Linear.int8_linear_backward": ["X8_3D", "SX16_3D", "G8_3D", "SG16_3D", "G8T", "W8", "SW16", "B", "stochastic",
                                    "dgrad_quantize"],
    "Nonlinear.int8_quantize": ["x", "QB", "stochastic"],
    "Nonlinear.int8_quantize_transpose": ["x", "QB", "stochastic", "transpose_output_2d"],
    "Nonlinear.int8_transpose": ["x", "transpose_output_2d"],
    "Nonlinear.int8_dequantize": ["x", "s_x", "QB"],
    "Nonlinear.int8_layernorm_forward": ["x", "sx", "weight", "mean", "rstd", "QB", "eps"],
    "Nonlinear.int8_layernorm_backward": ["x", "sx", "g", "sg", "w", "QB", "m", "v", "stochastic", "eps"],
    "Nonlinear.int8_gelu_forward": ["x", "s_x", "QB"],
    "Nonlinear.int8_gelu_backward": ["x", "s_x", "g", "s_g", "QB", "stochastic"],
    "Nonlinear.int8_add_Ifp_Ig16_Ofp_Og": ["x1", "x2", "s_x2", "QB", "stochastic"],
    "Nonlinear.int8_add_Ifp_Ig16_Ofp_Og_MeanVar": ["x1", "x2", "s_x2", "QB"],
}


@pytest.mark.parametrize("qual,params", SIGNATURES.items())
def test_signatures(qual, params):
    import importlib
    mod, fn = qual.split(".")
    f = getattr(importlib.import_module(mod), fn)
    got = list(inspect.signature(f).parameters)
    assert got[:len(params)] == params
    for extra in got[len(params):]:                 # anything we add must be optional
        assert inspect.signature(f).parameters[extra].default is not inspect.Parameter.empty


def test_cpu_tensors_are_rejected_not_computed():
    """No CPU fallback: host tensors raise."""
    import BlockQuantizeCUDA as BQC
    from Nonlinear import int8_gelu_forward, int8_quantize
    x = torch.randn(32, 32)
    with pytest.raises(RuntimeError, match="GPU"):
        int8_quantize(x, 32)
    with pytest.raises(RuntimeError, match="GPU"):
        int8_gelu_forward(torch.zeros(32, 32, dtype=torch.int8), torch.ones(1, 1, dtype=torch.float16), 32)
    with pytest.raises(RuntimeError, match="32"):
        int8_quantize(x, 16)
    a = torch.zeros(32, 32, dtype=torch.int8)
    s = torch.ones(1, 1, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU"):
        BQC.igemm_output_int_quantize(a, a, s, s, 32, 32, 32)
    with pytest.raises(RuntimeError, match="multiples of 32"):
        BQC.igemm_basic_int8_gemm(a, a, 32, 48, 32)
    with pytest.raises(RuntimeError, match="not implemented"):
        BQC.igemm_output_int_quantize_fused(a, a, s, s, 32, 32, 32)


# ------------------------------------------------------------------------------------------- GPU side
def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def eq(got, want):
    got = got.cpu().numpy()
    if got.dtype == np.float16:
        return np.array_equal(got.view(np.uint16), np.asarray(want, np.float16).view(np.uint16))
    return np.array_equal(got, want)


@pytest.mark.gpu
def test_bqc_functions_match_oracle(oracle):
    """Layouts as the reference's test scripts build them: sx [m/b,k/b] passed as sx.t().contiguous(),
    sw [k/b,n/b] passed as is (JetfireGEMMKernel/tests/test_int8igemmoutputIntQuantizeStochastic.py:24-41)."""
    import BlockQuantizeCUDA as BQC
    rng = np.random.default_rng(0)
    m, n, k = 128, 256, 96
    qx, qw = rand_codes(rng, (m, k)), rand_codes(rng, (k, n))
    sx, sw = rand_scales(rng, (m // QB, k // QB)), rand_scales(rng, (k // QB, n // QB))
    sxT = np.ascontiguousarray(sx.T)
    dqx, dqw = dev(qx), dev(qw)
    dsxT, dsw = dev(sxT.astype(np.float16)), dev(sw.astype(np.float16))

    assert eq(BQC.igemm_basic_int8_gemm(dqx, dqw, m, n, k), oracle.igemm_s32(qx, qw, 1))
    out = BQC.igemm_output_fp_no_quantize(dqx, dqw, dsxT, dsw, m, n, k)
    assert out.dtype == torch.float16 and eq(out, oracle.igemm_block_fp(qx, qw, sxT, sw, 1, "f16"))
    o, so = BQC.igemm_output_int_quantize(dqx, dqw, dsxT, dsw, m, n, k)
    wq, ws = oracle.igemm_block_q(qx, qw, sxT, sw, 1, scale_dtype="f16")
    assert o.dtype == torch.int8 and so.dtype == torch.float16 and tuple(so.shape) == (m // QB, n // QB)
    assert eq(o, wq) and eq(so, ws)

    torch.manual_seed(1234)
    BQC.philox_set_offset(0, 40)
    seed, offset = BQC.philox_peek(0)
    assert (seed, offset) == (1234, 40)
    o, so = BQC.igemm_output_int_quantize_stochastic(dqx, dqw, dsxT, dsw, m, n, k)
    wq, ws = oracle.igemm_block_q(qx, qw, sxT, sw, 1, stochastic=True, seed=seed, offset=offset, scale_dtype="f16")
    assert eq(o, wq) and eq(so, ws)
    assert BQC.philox_peek(0) == (1234, 40 + m * n // 8)
    o2, _ = BQC.igemm_output_int_quantize_stochastic(dqx, dqw, dsxT, dsw, m, n, k)
    assert not torch.equal(o, o2)                    # fresh noise on every call

    bias = (0.05 * rng.standard_normal(n)).astype(np.float32)
    biasmax = np.array([np.abs(bias).max()], np.float32)
    wq, ws = oracle.igemm_block_q(qx, qw, sxT, sw, 1, bias=bias, biasmax=float(biasmax[0]), scale_dtype="f16")
    o, so = BQC.igemm_output_int_quantize_bias_rowrow(dqx, dqw, dev(bias), dev(biasmax), dsxT, dsw, m, n, k)
    assert eq(o, wq) and eq(so, ws)
    # row x col: W stored [n,k], passed as its .t() view (JetfireGEMMKernel/tests/…BiasRowCol.py:38-40)
    w_nk = dev(np.ascontiguousarray(qw.T))
    view = w_nk.t()
    assert not view.is_contiguous()
    o, so = BQC.igemm_output_int_quantize_bias_rowcol(dqx, view, dev(bias), dev(biasmax), dsxT, dsw, m, n, k)
    assert eq(o, wq) and eq(so, ws)
    h = BQC.hgemm_v1(dqx.half(), dqw.half(), m, n, k)
    assert h.dtype == torch.float16 and tuple(h.shape) == (m, n)


@pytest.mark.gpu
def test_bqc_error_paths():
    import BlockQuantizeCUDA as BQC
    a = torch.zeros(64, 64, dtype=torch.int8, device="cuda")
    s = torch.ones(2, 2, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="int8"):
        BQC.igemm_output_int_quantize(a.float(), a, s, s, 64, 64, 64)
    with pytest.raises(RuntimeError, match="SX must be"):
        BQC.igemm_output_int_quantize(a, a, s[:1], s, 64, 64, 64)
    with pytest.raises(RuntimeError, match="same dtype"):
        BQC.igemm_output_int_quantize(a, a, s, s.float(), 64, 64, 64)
    with pytest.raises(RuntimeError, match="contiguous"):
        BQC.igemm_output_int_quantize(a, a.t(), s, s, 64, 64, 64)
    with pytest.raises(RuntimeError, match="same GPU"):
        BQC.igemm_output_int_quantize(a, a.cpu(), s, s, 64, 64, 64)
    with pytest.raises(RuntimeError, match=r"\[M,K\]"):
        BQC.igemm_output_int_quantize(a, a, s, s, 32, 64, 64)


@pytest.mark.gpu
def test_linear_package_3d_shapes_and_values(oracle):
    from Linear import int8_linear_backward, int8_linear_forward
    from Nonlinear import int8_dequantize, int8_quantize, int8_quantize_transpose, int8_transpose
    import BlockQuantizeCUDA as BQC
    torch.manual_seed(7)
    BS, T, Cin, Cout = 2, 64, 96, 160
    x = torch.randn(BS, T, Cin, device="cuda")
    w = torch.randn(Cout, Cin, device="cuda") * 0.02
    g = torch.randn(BS, T, Cout, device="cuda", dtype=torch.float16) * 1e-3
    qx, sx = int8_quantize(x, 32)
    qw, sw = int8_quantize(w, 32)
    assert tuple(qx.shape) == (BS, T, Cin) and tuple(sx.shape) == (BS, T // 32, Cin // 32) and sx.dtype == torch.float16
    o8, so = int8_linear_forward(qx, sx, qw, sw, True, 32)
    assert tuple(o8.shape) == (BS, T, Cout) and tuple(so.shape) == (BS, T // 32, Cout // 32)
    sx2 = sx.reshape(-1, Cin // 32)
    wq, ws = oracle.igemm_block_q(qx.reshape(-1, Cin).cpu().numpy(), qw.cpu().numpy(),
                                  np.ascontiguousarray(sx2.float().cpu().numpy().T),
                                  np.ascontiguousarray(sw.float().cpu().numpy().T), 0, scale_dtype="f16")
    assert eq(o8.reshape(-1, Cout), wq) and eq(so.reshape(-1, Cout // 32), ws)
    ofp = int8_linear_forward(qx, sx, qw, sw, False, 32)
    assert ofp.dtype == torch.float16 and tuple(ofp.shape) == (BS, T, Cout)
    assert torch.equal(ofp, int8_dequantize(o8, so, 32).half())
    ref = x.reshape(-1, Cin) @ w.t()
    assert torch.nn.functional.cosine_similarity(ofp.reshape(-1).float(), ref.reshape(-1), dim=0) > 0.999

    from Linear import int8_linear_forward_gelu
    from Nonlinear import int8_gelu_forward
    for approximate in ("none", "tanh"):
        f8, fs, fg8, fgs = int8_linear_forward_gelu(qx, sx, qw, sw, 32, approximate)
        g8, gs = int8_gelu_forward(o8, so, 32, approximate)
        assert torch.equal(f8, o8) and torch.equal(fs, so) and torch.equal(fg8, g8) and torch.equal(fgs, gs)

    qg, sg, qgt = int8_quantize_transpose(g, 32, stochastic=True, transpose_output_2d=True)
    assert tuple(qgt.shape) == (Cout, BS * T)
    assert torch.equal(qgt, int8_transpose(qg, transpose_output_2d=True))
    seed, off = BQC.philox_peek(0)
    gx8, gsx, gw = int8_linear_backward(qx, sx, qg, sg, qgt, qw, sw, 32, stochastic=True)
    assert tuple(gx8.shape) == (BS, T, Cin) and tuple(gsx.shape) == (BS, T // 32, Cin // 32)
    assert tuple(gw.shape) == (Cout, Cin) and gw.dtype == torch.float16
    sg2 = sg.reshape(-1, Cout // 32).float().cpu().numpy()
    wq, ws = oracle.igemm_block_q(qg.reshape(-1, Cout).cpu().numpy(), qw.cpu().numpy(), np.ascontiguousarray(sg2.T),
                                  sw.float().cpu().numpy(), 1, stochastic=True, seed=seed, offset=off, scale_dtype="f16")
    assert eq(gx8.reshape(-1, Cin), wq) and eq(gsx.reshape(-1, Cin // 32), ws)
    wgw = oracle.igemm_block_fp(qgt.cpu().numpy(), qx.reshape(-1, Cin).cpu().numpy(), sg2, sx2.float().cpu().numpy(), 1, "f16")
    assert eq(gw, wgw)
    seed2, off2 = BQC.philox_peek(0)
    gx, gw2 = int8_linear_backward(qx, sx, qg, sg, qgt, qw, sw, 32, stochastic=True, dgrad_quantize=False)
    assert gx.dtype == torch.float16 and tuple(gx.shape) == (BS, T, Cin) and torch.equal(gw2, gw)
    # the unquantised activation gradient = codes x scales of the stochastic requantisation drawn at (seed2, off2)
    wq2, ws2 = oracle.igemm_block_q(qg.reshape(-1, Cout).cpu().numpy(), qw.cpu().numpy(), np.ascontiguousarray(sg2.T),
                                    sw.float().cpu().numpy(), 1, stochastic=True, seed=seed2, offset=off2, scale_dtype="f16")
    want_gx = (wq2.astype(np.float32).reshape(BS * T // 32, 32, Cin // 32, 32)
               * ws2.astype(np.float32)[:, None, :, None]).reshape(BS * T, Cin).astype(np.float16)
    assert eq(gx.reshape(-1, Cin), want_gx)
    # without a materialised transpose: G8T=None, or the .t() view of the gradient handed to the extension
    _, gw3 = int8_linear_backward(qx, sx, qg, sg, None, qw, sw, 32, stochastic=True, dgrad_quantize=False)
    gw4 = BQC.igemm_output_fp_no_quantize(qg.reshape(-1, Cout).t(), qx.reshape(-1, Cin), sg.reshape(-1, Cout // 32),
                                          sx2, Cout, Cin, BS * T)
    assert torch.equal(gw3, gw) and torch.equal(gw4, gw)
    with pytest.raises(RuntimeError, match="contiguous or the .t\\(\\) view"):
        BQC.igemm_output_fp_no_quantize(qgt[:, ::2], qx.reshape(-1, Cin)[: BS * T // 2], sg.reshape(-1, Cout // 32)[: BS * T // 64],
                                        sx2[: BS * T // 64], Cout, Cin, BS * T // 2)
    ref_gx = g.reshape(-1, Cout).float() @ w
    assert torch.nn.functional.cosine_similarity(gx.reshape(-1).float(), ref_gx.reshape(-1), dim=0) > 0.99
    ref_gw = g.reshape(-1, Cout).float().t() @ x.reshape(-1, Cin)
    assert torch.nn.functional.cosine_similarity(gw.reshape(-1).float(), ref_gw.reshape(-1), dim=0) > 0.999


@pytest.mark.gpu
def test_weight_gradient_k_split_through_the_packages(oracle):
    """The K split of the weight gradient (an extension: trailing argument / keyword, default = the reference's single
    chain) through BlockQuantizeCUDA and Linear: bit-exact against the oracle's composition with the library's plan."""
    from Linear import int8_linear_backward
    from Nonlinear import int8_quantize
    import BlockQuantizeCUDA as BQC
    import jetfire_hip as jf
    torch.manual_seed(11)
    BS, T, Cin, Cout = 2, 1024, 96, 160
    x = torch.randn(BS, T, Cin, device="cuda")
    w = torch.randn(Cout, Cin, device="cuda") * 0.02
    g = torch.randn(BS, T, Cout, device="cuda", dtype=torch.float16) * 1e-3
    qx, sx = int8_quantize(x, 32)
    qw, sw = int8_quantize(w, 32)
    qg, sg = int8_quantize(g, 32, stochastic=True)
    K = BS * T
    A = np.ascontiguousarray(qg.reshape(K, Cout).cpu().numpy().T)
    X = qx.reshape(K, Cin).cpu().numpy()
    SG, SX = sg.reshape(-1, Cout // 32).float().cpu().numpy(), sx.reshape(-1, Cin // 32).float().cpu().numpy()
    for req in (2, 0):
        parts, per = jf.splitk_plan(Cout, Cin, K, req)
        assert parts > 1
        want = oracle.igemm_block_f32_splitk(A, X, SG, SX, 1, parts, per).astype(np.float16)
        got = BQC.igemm_output_fp_no_quantize(qg.reshape(K, Cout).t(), qx.reshape(K, Cin), sg.reshape(-1, Cout // 32),
                                              sx.reshape(-1, Cin // 32), Cout, Cin, K, req)
        assert eq(got, want)
    _, _, gw0 = int8_linear_backward(qx, sx, qg, sg, None, qw, sw, 32, wgrad_splitk=0)
    assert eq(gw0, want)
    _, _, gw1 = int8_linear_backward(qx, sx, qg, sg, None, qw, sw, 32)
    assert eq(gw1, oracle.igemm_block_fp(A, X, SG, SX, 1, "f16"))
    assert torch.allclose(gw0.float(), gw1.float(), rtol=2e-3, atol=1e-7)


@pytest.mark.gpu
def test_nonlinear_package_3d(oracle):
    from Nonlinear import (int8_add_Ifp_Ig16_Ofp_Og, int8_add_Ifp_Ig16_Ofp_Og_MeanVar, int8_dequantize,
                           int8_gelu_backward, int8_gelu_forward, int8_layernorm_backward, int8_layernorm_forward,
                           int8_quantize, int8_rowstats, int8_transpose)
    torch.manual_seed(3)
    BS, T, C = 2, 64, 160
    x = torch.randn(BS, T, C, device="cuda")
    res = torch.randn(BS, T, C, device="cuda").bfloat16()
    w = (1 + 0.1 * torch.randn(C, device="cuda"))
    qx, sx = int8_quantize(x, 32)
    fp, q2, s2, mean, rstd = int8_add_Ifp_Ig16_Ofp_Og_MeanVar(res, qx, sx, 32)
    assert fp.dtype == torch.float32 and tuple(fp.shape) == (BS, T, C) and tuple(mean.shape) == (BS, T)
    want = res.float() + int8_dequantize(qx, sx, 32)
    assert torch.equal(fp, want)
    assert torch.allclose(mean, want.mean(-1), atol=1e-5) and torch.allclose(rstd, want.var(-1, unbiased=False).rsqrt(), rtol=1e-4)
    qy, sy, (m_, r_) = int8_layernorm_forward(q2, s2, w, mean, rstd, 32)
    assert tuple(qy.shape) == (BS, T, C) and tuple(sy.shape) == (BS, T // 32, C // 32) and m_ is mean
    y_ref = torch.nn.functional.layer_norm(int8_dequantize(q2, s2, 32), (C,), w, None, 0.0)
    assert torch.nn.functional.cosine_similarity(int8_dequantize(qy, sy, 32).reshape(-1), y_ref.reshape(-1), dim=0) > 0.999
    qy2, sy2, (m2, r2) = int8_layernorm_forward(q2, s2, w, None, None, 32, eps=1e-5)     # statistics computed here
    assert tuple(m2.shape) == (BS, T)
    ms, rs = int8_rowstats(q2, s2, 32, 1e-5)
    assert torch.equal(ms, m2)
    g = torch.randn(BS, T, C, device="cuda") * 1e-3
    qg, sg = int8_quantize(g, 32, stochastic=True)
    qd, sd, dw = int8_layernorm_backward(q2, s2, qg, sg, w, 32, mean, rstd, stochastic=True)
    assert tuple(qd.shape) == (BS, T, C) and tuple(dw.shape) == (C,) and dw.dtype == w.dtype
    qh, sh = int8_gelu_forward(qx, sx, 32)
    assert tuple(qh.shape) == (BS, T, C)
    ref = torch.nn.functional.gelu(int8_dequantize(qx, sx, 32))
    assert torch.nn.functional.cosine_similarity(int8_dequantize(qh, sh, 32).reshape(-1), ref.reshape(-1), dim=0) > 0.999
    qb, sb = int8_gelu_backward(qx, sx, qg, sg, 32, stochastic=True)
    assert tuple(qb.shape) == (BS, T, C) and sb.dtype == torch.float16
    fpg, qa, sa = int8_add_Ifp_Ig16_Ofp_Og(g, qb, sb, 32, stochastic=True)
    assert fpg.dtype == torch.float32 and tuple(qa.shape) == (BS, T, C)
    t2 = int8_transpose(qx, transpose_output_2d=True)
    assert tuple(t2.shape) == (C, BS * T)
    t3 = int8_transpose(qx)
    assert t3.dim() == 3 and t3.shape[0] == BS and t3.shape[-1] == BS * T     # 3-D when not asked for 2-D


@pytest.mark.gpu
def test_stochastic_ops_share_one_counter_source(oracle):
    """The Nonlinear operators (ctypes binding) and the GEMM extension reserve their Philox counters from the same place,
    the device's torch generator: consecutive stochastic ops of a backward pass get disjoint counter ranges, and
    torch.manual_seed rewinds them, also when called with the seed that is already set."""
    from Linear import int8_linear_backward
    from Nonlinear import int8_gelu_backward, int8_quantize
    import BlockQuantizeCUDA as BQC
    import jetfire_hip as jf
    BS, T, Cin, Cout = 1, 256, 96, 160
    gsrc = torch.Generator().manual_seed(5)
    x = torch.randn(BS, T, Cin, generator=gsrc).cuda()
    w = (torch.randn(Cout, Cin, generator=gsrc) * 0.02).cuda()
    g = (torch.randn(BS, T, Cout, generator=gsrc) * 1e-3).cuda()
    qx, sx = int8_quantize(x, 32)
    qw, sw = int8_quantize(w, 32)

    def backward():
        spans = []
        seed, off = BQC.philox_peek(0)
        qg, sg = int8_quantize(g, 32, stochastic=True)             # Nonlinear: counters [off, off + T*Cout/8)
        spans.append((off, T * Cout // 8))
        assert jf.philox.peek(qg.device) == BQC.philox_peek(0)     # both bindings look at the same state
        seed2, off2 = BQC.philox_peek(0)
        gx8, gsx, gw = int8_linear_backward(qx, sx, qg, sg, None, qw, sw, 32)   # extension: the dgrad GEMM
        spans.append((off2, T * Cin // 8))
        seed3, off3 = BQC.philox_peek(0)
        d8, ds = int8_gelu_backward(gx8, gsx, gx8, gsx, 32, stochastic=True)    # Nonlinear again
        spans.append((off3, T * Cin // 8))
        assert seed == seed2 == seed3
        return spans, (qg, sg, gx8, gsx, d8, ds), (seed, off, off2)

    torch.manual_seed(77)
    spans, first, (seed, off, off2) = backward()
    assert seed == 77 and off == 0
    for (a, n), (b, _) in zip(spans, spans[1:]):
        assert b >= a + n, f"counter ranges overlap: {spans}"
    # each op used exactly the counters it reserved: the oracle reproduces it from (seed, offset)
    wq, ws = oracle.quantize(g.reshape(-1, Cout).cpu().numpy(), stochastic=True, seed=seed, offset=off, scale_dtype="f16")
    assert np.array_equal(first[0].reshape(-1, Cout).cpu().numpy(), wq)
    sg2 = first[1].reshape(-1, Cout // 32).float().cpu().numpy()
    wq, ws = oracle.igemm_block_q(first[0].reshape(-1, Cout).cpu().numpy(), qw.cpu().numpy(), np.ascontiguousarray(sg2.T),
                                  sw.float().cpu().numpy(), 1, stochastic=True, seed=seed, offset=off2, scale_dtype="f16")
    assert np.array_equal(first[2].reshape(-1, Cin).cpu().numpy(), wq)
    second_spans, second, _ = backward()                          # no re-seed: fresh counters, different noise
    assert second_spans[0][0] >= spans[-1][0] + spans[-1][1]
    assert not torch.equal(second[0], first[0])
    torch.manual_seed(77)                                          # same seed again: the stream rewinds
    again_spans, again, _ = backward()
    assert again_spans == spans
    for a, b in zip(first, again):
        assert torch.equal(a, b)


@pytest.mark.gpu
def test_linear_backward_with_fused_gelu_backward():
    """Linear.int8_linear_backward_gelu = int8_linear_backward then int8_gelu_backward, bit for bit, when both start
    from the same generator state (the fused kernel draws its two noise streams in the order of the two calls)."""
    from Linear import int8_linear_backward, int8_linear_backward_gelu
    from Nonlinear import int8_gelu_backward, int8_quantize
    BS, T, Cin, Cout = 2, 128, 160, 96
    gsrc = torch.Generator().manual_seed(9)
    pre = torch.randn(BS, T, Cin, generator=gsrc).cuda()                  # the GELU's input
    act = torch.nn.functional.gelu(pre)                                   # the linear layer's input
    w = (torch.randn(Cout, Cin, generator=gsrc) * 0.02).cuda()
    g = (torch.randn(BS, T, Cout, generator=gsrc) * 1e-3).cuda()
    qp, sp = int8_quantize(pre, 32)
    qa, sa = int8_quantize(act, 32)
    qw, sw = int8_quantize(w, 32)
    qg, sg = int8_quantize(g, 32)
    for approximate in ("none", "tanh"):
        torch.manual_seed(31)
        gx8, gsx, gw = int8_linear_backward(qa, sa, qg, sg, None, qw, sw, 32, stochastic=True, wgrad_splitk=0)
        d8, ds = int8_gelu_backward(qp, sp, gx8, gsx, 32, stochastic=True, approximate=approximate)
        torch.manual_seed(31)
        f8, fs, fw = int8_linear_backward_gelu(qa, sa, qg, sg, qw, sw, qp, sp, 32, approximate=approximate, stochastic=True,
                                               wgrad_splitk=0)
        assert tuple(f8.shape) == (BS, T, Cin) and tuple(fs.shape) == (BS, T // 32, Cin // 32)
        assert torch.equal(f8, d8) and torch.equal(fs, ds) and torch.equal(fw, gw)


@pytest.mark.gpu
def test_linear_package_with_bias(oracle):
    """bias through the Linear functions (sketched in the reference, QBlockLinear.py:38-39, 63-66): the forward adds it in
    the requantising epilogue with biasmax = max|bias| (…BiasRowCol.cu:313,357), bit-exact against the oracle; the GELU
    and dequantising epilogues take it as well; the backward returns the bias gradient = column sums of the gradient."""
    from Linear import int8_linear_backward, int8_linear_backward_gelu, int8_linear_forward, int8_linear_forward_gelu
    from Nonlinear import int8_column_sums, int8_dequantize, int8_gelu_forward, int8_quantize
    torch.manual_seed(17)
    BS, T, Cin, Cout = 2, 96, 160, 224
    x = torch.randn(BS, T, Cin, device="cuda")
    w = torch.randn(Cout, Cin, device="cuda") * 0.02
    bias = torch.randn(Cout, device="cuda") * 0.3
    g = torch.randn(BS, T, Cout, device="cuda") * 1e-3
    qx, sx = int8_quantize(x, 32)
    qw, sw = int8_quantize(w, 32)
    o8, so = int8_linear_forward(qx, sx, qw, sw, True, 32, bias=bias)
    sx2 = sx.reshape(-1, Cin // 32)
    b = bias.cpu().numpy()
    wq, ws = oracle.igemm_block_q(qx.reshape(-1, Cin).cpu().numpy(), qw.cpu().numpy(),
                                  np.ascontiguousarray(sx2.float().cpu().numpy().T), np.ascontiguousarray(sw.float().cpu().numpy().T),
                                  0, bias=b, biasmax=float(np.abs(b).max()), scale_dtype="f16")
    assert eq(o8.reshape(-1, Cout), wq) and eq(so.reshape(-1, Cout // 32), ws)
    o8_nobias, _ = int8_linear_forward(qx, sx, qw, sw, True, 32)
    assert not torch.equal(o8, o8_nobias)
    ref = x.reshape(-1, Cin) @ w.t() + bias
    got = int8_dequantize(o8, so, 32).reshape(-1, Cout)
    assert torch.nn.functional.cosine_similarity(got.reshape(-1), ref.reshape(-1), dim=0) > 0.999
    # the unquantised output and the fused GELU see the same biased accumulator
    ofp = int8_linear_forward(qx, sx, qw, sw, False, 32, bias=bias)
    assert torch.equal(ofp, int8_dequantize(o8, so, 32).half())
    f8, fs, fg8, fgs = int8_linear_forward_gelu(qx, sx, qw, sw, 32, bias=bias)
    g8, gs = int8_gelu_forward(o8, so, 32)
    assert torch.equal(f8, o8) and torch.equal(fs, so) and torch.equal(fg8, g8) and torch.equal(fgs, gs)
    # bias gradient
    qg, sg = int8_quantize(g, 32, stochastic=True)
    torch.manual_seed(3)
    gx8, gsx, gw = int8_linear_backward(qx, sx, qg, sg, None, qw, sw, 32)
    torch.manual_seed(3)
    gx8b, gsxb, gwb, gb = int8_linear_backward(qx, sx, qg, sg, None, qw, sw, 32, bias_grad=True)
    assert torch.equal(gx8, gx8b) and torch.equal(gsx, gsxb) and torch.equal(gw, gwb)
    want = oracle.block_colsum(qg.reshape(-1, Cout).cpu().numpy(), sg.reshape(-1, Cout // 32).float().cpu().numpy())
    assert gb.dtype == torch.float32 and np.array_equal(gb.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert torch.equal(gb, int8_column_sums(qg, sg, 32))
    ref_gb = int8_dequantize(qg, sg, 32).reshape(-1, Cout).double().sum(0)
    assert torch.allclose(gb.double(), ref_gb, rtol=1e-4, atol=1e-7)
    out = int8_linear_backward(qx, sx, qg, sg, None, qw, sw, 32, dgrad_quantize=False, bias_grad=True)
    assert len(out) == 3 and torch.equal(out[2], gb)
    pre8, spre = int8_quantize(torch.randn(BS, T, Cin, device="cuda"), 32)
    out = int8_linear_backward_gelu(qx, sx, qg, sg, qw, sw, pre8, spre, 32, bias_grad=True)
    assert len(out) == 4 and torch.equal(out[3], gb)
    with pytest.raises(RuntimeError, match="elements"):
        int8_linear_forward(qx, sx, qw, sw, True, 32, bias=bias[:-1])


@pytest.mark.gpu
def test_packages_run_through_the_cpp_extension(oracle):
    """Every operator of Linear / Nonlinear is a function of the C++ extension (BlockQuantizeCUDA and its submodule
    `jetfire`): the ctypes binding of the C ABI, which the kernel tests use, gives the same bits on the same (seed, offset),
    and the extension rejects bad operands itself."""
    import BlockQuantizeCUDA as BQC
    import jetfire_hip as jf
    import Linear.linear as L
    import Nonlinear.ops as N
    J = BQC.jetfire
    assert N._jf is J and L._jf is J and L.BQC is BQC
    for mod in (N, L):
        assert "jetfire_hip" not in vars(mod), "the packages must not call the ctypes binding"
    torch.manual_seed(5)
    R, C = 128, 160
    x = torch.randn(R, C, device="cuda")
    q, s, qT = J.quantize(x, J.ROUND_STOCHASTIC, torch.float16, True, 0.0, 9, 4)
    q2, s2, qT2 = jf.quantize(x, jf.ROUND_STOCHASTIC, torch.float16, transpose=True, seed=9, offset=4)
    assert torch.equal(q, q2) and torch.equal(s, s2) and torch.equal(qT, qT2)
    g, sg, _ = J.quantize(torch.randn(R, C, device="cuda") * 1e-3, J.ROUND_NEAREST, torch.float16)
    a = J.gelu_bwd(q, s, g, sg, J.GELU_TANH, J.ROUND_STOCHASTIC, 3, 8)
    b = jf.gelu_bwd(q, s, g, sg, jf.GELU_TANH, jf.ROUND_STOCHASTIC, seed=3, offset=8)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    mean, rstd = J.rowstats(q, s, 1e-5)
    gamma = 1 + 0.1 * torch.randn(C, device="cuda")
    x1 = torch.randn(R, C, device="cuda").bfloat16()
    a = J.layernorm_bwd_add(q, s, g, sg, gamma, mean, rstd, x1, J.ROUND_STOCHASTIC, J.ROUND_STOCHASTIC_TRUNC, True, torch.bfloat16,
                            1, 0, 2, 4)
    b = jf.layernorm_bwd_add(q, s, g, sg, gamma, mean, rstd, x1, jf.ROUND_STOCHASTIC, jf.ROUND_STOCHASTIC_TRUNC, True, torch.bfloat16,
                             seed=1, offset=0, add_seed=2, add_offset=4)
    for u, v in zip(a, b):
        assert torch.equal(u, v)
    y1, qa, sa, m2, r2 = J.add(x1, q, s, J.ROUND_TRUNC, True, torch.float32)
    y1b, qab, sab, rs, rq = jf.add(x1, q, s, jf.ROUND_TRUNC, with_stats=True)
    mb, rb = jf.rowstats_finish(rs, rq, C)
    assert torch.equal(y1, y1b) and torch.equal(qa, qab) and torch.equal(m2, mb) and torch.equal(r2, rb)
    # no seed given: counters come from the device's generator, under its mutex, and advance
    torch.manual_seed(21)
    before = BQC.philox_peek(0)
    J.quantize(x, J.ROUND_STOCHASTIC)
    assert BQC.philox_peek(0) == (21, before[1] + R * C // 8)
    # operand errors are the extension's own
    with pytest.raises(RuntimeError, match="int8"):
        J.gelu_fwd(x, s)
    with pytest.raises(RuntimeError, match="scale shape"):
        J.gelu_fwd(q, s[:1])
    with pytest.raises(RuntimeError, match="rounding"):
        J.quantize(x, 7)
    with pytest.raises(RuntimeError, match="contiguous"):
        J.dequantize(q.t(), s)
    with pytest.raises(RuntimeError, match="float32 vector"):
        J.layernorm_fwd(q, s, gamma.half(), None, mean, rstd)
    with pytest.raises(RuntimeError, match="come together"):
        J.igemm_block_q(q, q, s.t(), s.t(), J.B_NK, gamma, None)


def test_expanded_gradient_is_copied_not_rejected():
    """int8_quantize_concat reads slabs where they lie only when their rows do not overlap: an expanded gradient (row stride
    0) is made contiguous first (CPU check of the rule; the tensors never reach a kernel here)."""
    import Nonlinear.ops as N
    seen = {}

    class Fake:
        ROUND_NEAREST, ROUND_STOCHASTIC = 0, 1

        @staticmethod
        def quantize_slabs(flat, rounding, scale_dtype):
            seen["flat"] = flat
            R = flat[0].shape[0]
            Ct = sum(f.shape[1] for f in flat)
            return torch.zeros(R, Ct, dtype=torch.int8), torch.zeros(R // 32, Ct // 32, dtype=scale_dtype)

    real = N._jf
    N._jf = Fake
    try:
        a = torch.randn(64, 32)
        b = torch.randn(1, 32).expand(64, 32)                       # stride (0, 1)
        c = torch.randn(64, 96)[:, 32:64]                            # a column slab of a wider tensor: read in place
        q, s = N.int8_quantize_concat([a, b, c], 32)
    finally:
        N._jf = real
    fa, fb, fc = seen["flat"]
    assert fb.stride(0) == 32 and fb.is_contiguous() and torch.equal(fb, b)
    assert fa.data_ptr() == a.data_ptr() and fc.data_ptr() == c.data_ptr() and fc.stride(0) == 96
    assert tuple(q.shape) == (64, 96) and tuple(s.shape) == (2, 3)
