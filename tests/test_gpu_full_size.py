"""The benchmark configurations at their full sizes, through the C ABI, against the CPU oracle.

Every kernel here is local to 32-row strips of its output (GEMM rows, block rows of the block-local kernels, LayerNorm
rows), so a strip of the output computed by the oracle from the matching strip of the inputs is a complete, bit-exact
check of that strip.  Each case checks three strips: the first, an interior one that does not start on a 128-row tile
boundary, and the last; all columns of each, so ragged last column tiles (1600, 4800 and 2304 are not multiples of the
128-wide tile) and every K depth are covered.  Bars as everywhere: codes, scales, INT32 and fp32 accumulators bit-exact.

Shapes (M, N, K) per layer: forward (T, C_out, C_in), dgrad (T, C_in, C_out), wgrad (C_out, C_in, T).
"""
import numpy as np
import pytest
import torch

from helpers import QB

pytestmark = pytest.mark.gpu


def same(got, want, what):
    got = got.cpu().numpy() if isinstance(got, torch.Tensor) else got
    if got.dtype == np.float16:
        g, w = got.view(np.uint16), want.view(np.uint16)
    elif got.dtype == np.float32:
        g, w = got.view(np.uint32), want.view(np.uint32)
    else:
        g, w = got, want
    assert g.shape == w.shape, f"{what}: shape {g.shape} vs {w.shape}"
    bad = np.argwhere(g != w)
    assert bad.shape[0] == 0, f"{what}: {bad.shape[0]} of {g.size} differ; first at {bad[0].tolist()}: " \
                              f"got {got[tuple(bad[0])]}, want {want[tuple(bad[0])]}"


def cont(a):
    return np.ascontiguousarray(a)


def strips(n):
    """First, an interior one off the 128 grid, last."""
    return (0, (n // 2 // QB) * QB - 32 if (n // 2) % 128 == 0 else (n // 2 // QB) * QB, n - QB)


def layer_inputs(T, Cin, Cout, seed, outliers):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, Cin, generator=g)
    if outliers:                                                   # 1 % of the channels x20
        idx = torch.randperm(Cin, generator=g)[: (Cin + 99) // 100]
        x[:, idx] *= 20
    w = torch.randn(Cout, Cin, generator=g) * 0.02
    dy = torch.randn(T, Cout, generator=g) * 1e-3
    return x, w, dy


def check_linear_layer(jf, oracle, T, Cin, Cout, seed, outliers, gelu=None, gelu_bwd=False):
    """forward (deterministic), dgrad (stochastic), wgrad (one chain from a transposed copy; and, as the recipe runs it,
    from the gradient in place with the library's K split) of one linear layer on quantised synthetic data."""
    print(f"layer T={T} {Cin}->{Cout} seed={seed}", flush=True)
    x, w, dy = layer_inputs(T, Cin, Cout, seed, outliers)
    f32 = torch.float32
    qx, sx = jf.quantize(x.cuda(), scale_dtype=f32)
    qw, sw = jf.quantize(w.cuda(), scale_dtype=f32)
    qg, sg, qgT = jf.quantize(dy.cuda(), rounding=jf.ROUND_STOCHASTIC, scale_dtype=f32, transpose=True, seed=seed, offset=0)
    del x, w, dy
    y, sy = jf.igemm_block_q(qx, qw, sx.t(), sw.t(), jf.B_NK)                       # scale operands read in place
    dx, sdx = jf.igemm_block_q(qg, qw, sg.t(), sw, jf.B_KN, rounding=jf.ROUND_STOCHASTIC, seed=seed + 1, offset=17)
    dw = jf.igemm_block_fp(qgT, qx, sg, sx, jf.B_KN, f32)
    parts, per = jf.splitk_plan(Cout, Cin, T, 0)
    dw_km = jf.igemm_block_fp(qg, qx, sg, sx, jf.B_KN, f32, a_layout=jf.A_KM, splitk=0)
    dw_km16 = jf.igemm_block_fp(qg, qx, sg, sx, jf.B_KN, torch.float16, a_layout=jf.A_KM, splitk=0)
    if gelu is not None:
        eps = 5e-5 if gelu == jf.GELU_ERF else 0.0
        fq, fs, fg, fgs = jf.igemm_block_q_gelu(qx, qw, sx.t(), sw.t(), gelu, eps)
        assert torch.equal(fq, y) and torch.equal(fs, sy), "fused forward differs from the plain forward"
        g2, gs2 = jf.gelu_fwd(y, sy, gelu, eps)
        assert torch.equal(fg, g2) and torch.equal(fgs, gs2), "fused GELU differs from the GELU kernel"
    if gelu_bwd:
        # this layer's input is the output of a GELU: its backward runs in the epilogue of the dgrad GEMM (the recipe's
        # MLP path); qx / sx stand in for the GELU's saved input, an [T, Cin] block tensor like the gradient
        fb, fbs = jf.igemm_block_q_gelu_bwd(qg, qw, sg.t(), sw, qx, sx, jf.GELU_ERF, jf.ROUND_STOCHASTIC, seed=seed + 1,
                                            offset=17, gelu_seed=seed + 2, gelu_offset=5)
        b2, bs2 = jf.gelu_bwd(qx, sx, dx, sdx, jf.GELU_ERF, jf.ROUND_STOCHASTIC, seed=seed + 2, offset=5)
        assert torch.equal(fb, b2) and torch.equal(fbs, bs2), "fused GELU backward differs from the GELU backward kernel"
    torch.cuda.synchronize()
    X, W, G, GT = (t.cpu().numpy() for t in (qx, qw, qg, qgT))
    SX, SW, SG = (t.cpu().numpy() for t in (sx, sw, sg))
    SWt = cont(SW.T)
    for r0 in strips(T):
        rows, rb = slice(r0, r0 + QB), slice(r0 // QB, r0 // QB + 1)
        wq, wsc = oracle.igemm_block_q(X[rows], W, cont(SX[rb].T), SWt, 0)
        same(y[rows], wq, f"forward codes rows {r0}")
        same(sy[rb], wsc, f"forward scales rows {r0}")
        if gelu is not None:
            wg, wgs = oracle.gelu_fwd(wq, wsc, gelu, eps)
            same(fg[rows], wg, f"fused GELU codes rows {r0}")
            same(fgs[rb], wgs, f"fused GELU scales rows {r0}")
        acc = oracle.igemm_block_f32(G[rows], W, cont(SG[rb].T), SW, 1)
        wq, wsc = oracle.requant(acc, stochastic=True, seed=seed + 1, offset=17 + r0 * Cin // 8)
        same(dx[rows], wq, f"dgrad codes rows {r0}")
        same(sdx[rb], wsc, f"dgrad scales rows {r0}")
        if gelu_bwd:
            wb, wbs = oracle.gelu_bwd(X[rows], SX[rb], wq, wsc, 0, True, seed + 2, 5 + r0 * Cin // 8)
            same(fb[rows], wb, f"fused GELU backward codes rows {r0}")
            same(fbs[rb], wbs, f"fused GELU backward scales rows {r0}")
    for r0 in strips(Cout):
        rows, rb = slice(r0, r0 + QB), slice(r0 // QB, r0 // QB + 1)
        sa = cont(SG[:, rb])
        same(dw[rows], oracle.igemm_block_f32(GT[rows], X, sa, SX, 1), f"wgrad rows {r0}")
        want = oracle.igemm_block_f32_splitk(GT[rows], X, sa, SX, 1, parts, per)
        same(dw_km[rows], want, f"wgrad in place, {parts} parts, rows {r0}")
        with np.errstate(over="ignore"):
            same(dw_km16[rows], want.astype(np.float16), f"wgrad in place fp16, rows {r0}")


def test_cfg1_cpu_path_case(jf, oracle):
    """2048 x 768 x 768, fp32 scales, seed 0, deterministic requantisation: every code, every scale and every per-K-block
    INT32 accumulator [24, 2048, 768]."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2048, 768, generator=g)
    w = torch.randn(768, 768, generator=g) * 0.02
    qx, sx = jf.quantize(x.cuda(), scale_dtype=torch.float32)
    qw, sw = jf.quantize(w.cuda(), scale_dtype=torch.float32)
    oqx, osx = oracle.quantize(x.numpy())
    oqw, osw = oracle.quantize(w.numpy())
    same(qx, oqx, "activation codes"); same(sx, osx, "activation scales")
    same(qw, oqw, "weight codes"); same(sw, osw, "weight scales")
    y, sy = jf.igemm_block_q(qx, qw, sx.t().contiguous(), sw.t().contiguous(), jf.B_NK)
    acc = jf.igemm_block_acc(qx, qw, jf.B_NK)
    wy, wsy = oracle.igemm_block_q(oqx, oqw, cont(osx.T), cont(osw.T), 0)
    same(y, wy, "output codes")
    same(sy, wsy, "output scales")
    wacc = oracle.igemm_block_acc(oqx, oqw, 0)
    assert wacc.shape == (24, 2048, 768) and np.abs(wacc).max() <= 32 * 127 * 127
    same(acc, wacc, "per-K-block INT32 accumulators")
    same(jf.igemm_s32(qx, qw, jf.B_NK), wacc.sum(axis=0, dtype=np.int64).astype(np.int32), "sum of the block accumulators")


@pytest.mark.parametrize("name,Cin,Cout", [("qkv", 768, 2304), ("proj", 768, 768), ("fc", 768, 3072), ("fc2", 3072, 768)])
def test_cfg2_gpt2_small_layer(jf, oracle, name, Cin, Cout):
    check_linear_layer(jf, oracle, 12288, Cin, Cout, seed=0, outliers=False)


@pytest.mark.parametrize("name,Cin,Cout,gelu", [("qkv", 1600, 4800, None), ("proj", 1600, 1600, None),
                                               ("fc", 1600, 6400, 0), ("fc2", 6400, 1600, None)])
def test_cfg3_gpt2_xl_layer(jf, oracle, name, Cin, Cout, gelu):
    """fc also runs the forward with the GELU fused into the epilogue, fc2 the activation gradient with the GELU
    backward fused into the epilogue (the recipe's MLP path)."""
    check_linear_layer(jf, oracle, 8192, Cin, Cout, seed=0, outliers=True, gelu=gelu, gelu_bwd=name == "fc2")


def test_cfg4_layernorm_full_size(jf, oracle):
    """LayerNorm forward and backward (stochastic rounding, dgamma, dbeta) on 8192 x 1600."""
    R, C = 8192, 1600
    g = torch.Generator().manual_seed(0)
    x = torch.randn(R, C, generator=g)
    gamma = 1 + 0.1 * torch.randn(C, generator=g)
    beta = 0.1 * torch.randn(C, generator=g)
    dy = 1e-3 * torch.randn(R, C, generator=g)
    f32 = torch.float32
    qx, sx = jf.quantize(x.cuda(), scale_dtype=f32)
    qg, sg = jf.quantize(dy.cuda(), jf.ROUND_STOCHASTIC, f32, seed=0, offset=0)
    mean, rstd = jf.rowstats(qx, sx, 1e-5)
    qy, sy = jf.layernorm_fwd(qx, sx, gamma.cuda(), beta.cuda(), mean, rstd)
    qd, sd, dg, db = jf.layernorm_bwd(qx, sx, qg, sg, gamma.cuda(), mean, rstd, jf.ROUND_STOCHASTIC, seed=4, offset=9)
    torch.cuda.synchronize()
    X, SX, G, SG = (t.cpu().numpy() for t in (qx, sx, qg, sg))
    gm, bt = gamma.numpy(), beta.numpy()
    M, RS = mean.cpu().numpy(), rstd.cpu().numpy()
    for r0 in strips(R):
        rows, rb = slice(r0, r0 + QB), slice(r0 // QB, r0 // QB + 1)
        wm, wr = oracle.rowstats(X[rows], SX[rb], 1e-5)
        same(M[rows], wm, f"mean rows {r0}")
        same(RS[rows], wr, f"rstd rows {r0}")
        wq, ws = oracle.layernorm_fwd(X[rows], SX[rb], gm, bt, wm, wr)
        same(qy[rows], wq, f"forward codes rows {r0}")
        same(sy[rb], ws, f"forward scales rows {r0}")
        wq, ws, _, _ = oracle.layernorm_bwd(X[rows], SX[rb], G[rows], SG[rb], gm, wm, wr, True, 4, 9 + r0 * C // 8)
        same(qd[rows], wq, f"backward codes rows {r0}")
        same(sd[rb], ws, f"backward scales rows {r0}")
    # dgamma / dbeta: sums over all 8192 rows, against float64
    xd = X.astype(np.float64) * np.repeat(np.repeat(SX.astype(np.float64), QB, 0), QB, 1)
    gd = G.astype(np.float64) * np.repeat(np.repeat(SG.astype(np.float64), QB, 0), QB, 1)
    xh = (xd - M[:, None].astype(np.float64)) * RS[:, None].astype(np.float64)
    wdg, wdb = (gd * xh).sum(0), gd.sum(0)
    assert np.allclose(dg.cpu().numpy(), wdg, rtol=1e-4, atol=1e-5 * np.abs(wdg).max())
    assert np.allclose(db.cpu().numpy(), wdb, rtol=1e-4, atol=1e-5 * np.abs(wdb).max())


@pytest.mark.parametrize("approx", [0, 1])
def test_cfg4_gelu_backward_full_size(jf, oracle, approx):
    """GELU backward (erf and tanh forms) with stochastic rounding on 8192 x 6400; forward in the erf form as well (the
    tanh forward is checked with the block-kernel tests)."""
    R, C = 8192, 6400
    g = torch.Generator().manual_seed(0)
    x = torch.randn(R, C, generator=g)
    dy = 1e-3 * torch.randn(R, C, generator=g)
    f32 = torch.float32
    qx, sx = jf.quantize(x.cuda(), scale_dtype=f32)
    qg, sg = jf.quantize(dy.cuda(), jf.ROUND_STOCHASTIC, f32, seed=0, offset=0)
    del x, dy
    qd, sd = jf.gelu_bwd(qx, sx, qg, sg, approx, jf.ROUND_STOCHASTIC, seed=6, offset=2)
    eps = 5e-5 if approx == 0 else 0.0
    qy, sy = jf.gelu_fwd(qx, sx, approx, eps)
    torch.cuda.synchronize()
    for r0 in strips(R):
        rows, rb = slice(r0, r0 + QB), slice(r0 // QB, r0 // QB + 1)
        X, SX, G, SG = (t.cpu().numpy() for t in (qx[rows], sx[rb], qg[rows], sg[rb]))
        wq, ws = oracle.gelu_bwd(X, SX, G, SG, approx, True, 6, 2 + r0 * C // 8)
        same(qd[rows], wq, f"backward codes rows {r0}")
        same(sd[rb], ws, f"backward scales rows {r0}")
        wq, ws = oracle.gelu_fwd(X, SX, approx, eps)
        same(qy[rows], wq, f"forward codes rows {r0}")
        same(sy[rb], ws, f"forward scales rows {r0}")
