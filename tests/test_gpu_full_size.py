"""The benchmark configurations at their full sizes, through the C ABI, against the CPU oracle.

The GEMMs are compared over their WHOLE outputs, bit for bit: which workgroup computes which tile (and which part of a
K split) depends on the shape of the launch, so a sample of rows would not notice a tile computed twice or not at all in
the rows it leaves out.  The oracle needs about half a second per GPT-2 XL GEMM on 16 host threads.  The block-local
kernels (LayerNorm, GELU) are compared over their whole outputs as well (about a second per tensor for the oracle).
Bars as everywhere: codes, scales, INT32 and fp32 accumulators bit-exact.

Shapes (M, N, K) per layer: forward (T, C_out, C_in), dgrad (T, C_in, C_out), wgrad (C_out, C_in, T).
"""
import numpy as np
import pytest
import torch

from helpers import QB, rand_codes, rand_scales

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
    # forward, every tile
    wq, wsc = oracle.igemm_block_q(X, W, cont(SX.T), cont(SW.T), 0)
    same(y, wq, "forward codes")
    same(sy, wsc, "forward scales")
    if gelu is not None:
        wg, wgs = oracle.gelu_fwd(wq, wsc, gelu, eps)
        same(fg, wg, "fused GELU codes")
        same(fgs, wgs, "fused GELU scales")
    # activation gradient, every tile
    acc = oracle.igemm_block_f32(G, W, cont(SG.T), SW, 1)
    wq, wsc = oracle.requant(acc, stochastic=True, seed=seed + 1, offset=17)
    del acc
    same(dx, wq, "dgrad codes")
    same(sdx, wsc, "dgrad scales")
    if gelu_bwd:
        wb, wbs = oracle.gelu_bwd(X, SX, wq, wsc, 0, True, seed + 2, 5)
        same(fb, wb, "fused GELU backward codes")
        same(fbs, wbs, "fused GELU backward scales")
    # weight gradient, every tile: one chain from the transposed copy, and the gradient in place with the library's K split
    same(dw, oracle.igemm_block_f32(GT, X, SG, SX, 1), "wgrad")
    want = oracle.igemm_block_f32_splitk(GT, X, SG, SX, 1, parts, per)
    same(dw_km, want, f"wgrad in place, {parts} parts")
    with np.errstate(over="ignore"):
        same(dw_km16, want.astype(np.float16), "wgrad in place fp16")


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


def test_cfg5_stress_cube(jf, oracle):
    """M = N = K = 8192, heavy-tailed A (Student-t, 3 degrees of freedom), B ~ N(0, 0.02); the requantised output in
    deterministic and in stochastic mode, every code and every scale."""
    n = 8192
    g = torch.Generator().manual_seed(0)
    a = torch.randn(n, n, generator=g) / torch.sqrt(torch.randn(3, n, n, generator=g).pow_(2).mean(0))   # t(3) = z / sqrt(chi2_3 / 3)
    b = torch.randn(n, n, generator=g) * 0.02
    qa, sa = jf.quantize(a.cuda(), scale_dtype=torch.float32)
    qb, sb = jf.quantize(b.cuda(), scale_dtype=torch.float32)
    del a, b
    print("cfg5 8192^3 deterministic + stochastic", flush=True)
    y, sy = jf.igemm_block_q(qa, qb, sa.t(), sb.t(), jf.B_NK)
    z, sz = jf.igemm_block_q(qa, qb, sa.t(), sb.t(), jf.B_NK, rounding=jf.ROUND_STOCHASTIC, seed=5, offset=11)
    torch.cuda.synchronize()
    A, B, SA, SB = (t.cpu().numpy() for t in (qa, qb, sa, sb))
    acc = oracle.igemm_block_f32(A, B, cont(SA.T), cont(SB.T), 0)
    wq, wsc = oracle.requant(acc)
    same(y, wq, "deterministic codes")
    same(sy, wsc, "deterministic scales")
    wq, wsc = oracle.requant(acc, stochastic=True, seed=5, offset=11)
    same(z, wq, "stochastic codes")
    same(sz, wsc, "stochastic scales")


# One odd-shaped launch per regime of the launcher's choice of wave priorities (by the number of 128 x 128 workgroups
# against the 512 that are resident at once: up to one round; 1 to 1.5 rounds with short and with long tiles; 1.5 to 2;
# more than 2), each with a number of tile rows that is not a multiple of the 8-row groups the tile order walks, a
# workgroup count that is not a multiple of the 8 XCDs, and ragged last tiles in both directions.
PACE_SHAPES = [
    (11 * 128 - 32, 13 * 128 - 64, 512),        # 143 workgroups
    (21 * 128 - 32, 29 * 128 - 96, 256),        # 609: 1.19 rounds, short tiles
    (21 * 128 - 32, 29 * 128 - 96, 4096),       # 609: long tiles
    (27 * 128 - 64, 33 * 128 - 32, 384),        # 891: 1.74 rounds
    (37 * 128 - 96, 31 * 128 - 64, 160),        # 1147: 2.24 rounds
]


@pytest.mark.parametrize("M,N,K", PACE_SHAPES)
@pytest.mark.parametrize("layout", [0, 1])
def test_odd_shapes_in_every_pacing_regime(jf, oracle, M, N, K, layout):
    tiles = ((M + 127) // 128) * ((N + 127) // 128)
    assert tiles % 8 and ((M + 127) // 128) % 8
    print(f"odd shape M={M} N={N} K={K} layout={layout} workgroups={tiles}", flush=True)
    rng = np.random.default_rng(M + N + K + layout)
    A = rand_codes(rng, (M, K))
    B = rand_codes(rng, (K, N) if layout else (N, K))
    sa = rand_scales(rng, (K // QB, M // QB), f16=False)
    sb = rand_scales(rng, (K // QB, N // QB), f16=False)
    dA, dB, dsa, dsb = (torch.from_numpy(t).cuda() for t in (A, B, sa, sb))
    q, sc = jf.igemm_block_q(dA, dB, dsa, dsb, layout)
    z, sz = jf.igemm_block_q(dA, dB, dsa, dsb, layout, rounding=jf.ROUND_STOCHASTIC, seed=9, offset=3)
    fp = jf.igemm_block_fp(dA, dB, dsa, dsb, layout, torch.float32)
    torch.cuda.synchronize()
    acc = oracle.igemm_block_f32(A, B, sa, sb, layout)
    same(fp, acc, "fp32 accumulators")
    wq, wsc = oracle.requant(acc)
    same(q, wq, "deterministic codes"); same(sc, wsc, "deterministic scales")
    wq, wsc = oracle.requant(acc, stochastic=True, seed=9, offset=3)
    same(z, wq, "stochastic codes"); same(sz, wsc, "stochastic scales")


@pytest.mark.parametrize("M,N,K,req", [(11 * 128 - 32, 5 * 128 - 96, 4096, 0), (3 * 128, 7 * 128 - 32, 6144, 5),
                                       (13 * 128 - 64, 3 * 128 - 32, 2048, 3)])
def test_odd_shapes_with_a_k_split(jf, oracle, M, N, K, req):
    """The weight-gradient form (A given as [K,M], B as [K,N]) with several parts: workgroups are ordered part-major
    over the same tile map, every part of every tile must be computed exactly once."""
    parts, per = jf.splitk_plan(M, N, K, req)
    assert parts > 1 and (req == 0 or (parts * ((M + 127) // 128) * ((N + 127) // 128)) % 8)
    print(f"odd split shape M={M} N={N} K={K} parts={parts}", flush=True)
    rng = np.random.default_rng(M + N + K)
    At = rand_codes(rng, (K, M))
    B = rand_codes(rng, (K, N))
    sa = rand_scales(rng, (K // QB, M // QB), f16=False)
    sb = rand_scales(rng, (K // QB, N // QB), f16=False)
    dA, dB, dsa, dsb = (torch.from_numpy(t).cuda() for t in (At, B, sa, sb))
    got = jf.igemm_block_fp(dA, dB, dsa, dsb, jf.B_KN, torch.float32, a_layout=jf.A_KM, splitk=req)
    torch.cuda.synchronize()
    same(got, oracle.igemm_block_f32_splitk(cont(At.T), B, sa, sb, 1, parts, per), f"{parts} parts")


def test_cfg4_layernorm_full_size(jf, oracle):
    """LayerNorm statistics, forward and backward (stochastic rounding, dgamma, dbeta) on 8192 x 1600, whole outputs."""
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
    # the whole tensors (the oracle takes a second or two for them)
    wm, wr = oracle.rowstats(X, SX, 1e-5)
    same(M, wm, "mean")
    same(RS, wr, "rstd")
    wq, ws = oracle.layernorm_fwd(X, SX, gm, bt, wm, wr)
    same(qy, wq, "forward codes")
    same(sy, ws, "forward scales")
    wq, ws, _, _ = oracle.layernorm_bwd(X, SX, G, SG, gm, wm, wr, True, 4, 9)
    same(qd, wq, "backward codes")
    same(sd, ws, "backward scales")
    # dgamma / dbeta: sums over all 8192 rows, against float64
    xd = X.astype(np.float64) * np.repeat(np.repeat(SX.astype(np.float64), QB, 0), QB, 1)
    gd = G.astype(np.float64) * np.repeat(np.repeat(SG.astype(np.float64), QB, 0), QB, 1)
    xh = (xd - M[:, None].astype(np.float64)) * RS[:, None].astype(np.float64)
    wdg, wdb = (gd * xh).sum(0), gd.sum(0)
    assert np.allclose(dg.cpu().numpy(), wdg, rtol=1e-4, atol=1e-5 * np.abs(wdg).max())
    assert np.allclose(db.cpu().numpy(), wdb, rtol=1e-4, atol=1e-5 * np.abs(wdb).max())


@pytest.mark.parametrize("approx", [0, 1])
def test_cfg4_gelu_backward_full_size(jf, oracle, approx):
    """GELU backward and forward (erf and tanh forms; backward with stochastic rounding) on 8192 x 6400, whole outputs."""
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
    X, SX, G, SG = (t.cpu().numpy() for t in (qx, sx, qg, sg))     # the whole tensors: about a second each for the oracle
    wq, ws = oracle.gelu_bwd(X, SX, G, SG, approx, True, 6, 2)
    same(qd, wq, "backward codes")
    same(sd, ws, "backward scales")
    wq, ws = oracle.gelu_fwd(X, SX, approx, eps)
    same(qy, wq, "forward codes")
    same(sy, ws, "forward scales")


@pytest.mark.parametrize("approx", [0, 1])
def test_gelu_whole_output_against_row_slices_and_more_groups_than_waves(jf, oracle, approx):
    """A wave of the GELU kernels takes a group of four adjacent blocks, and at most 16384 waves are launched: 8192 x 8352
    has 256 x 66 = 16896 groups (the last group of a row is a single block), so some waves take a second group.  The
    whole outputs must equal what the same kernels give on 512-row slices (1056 groups each; the noise of a slice is
    that of its rows in the whole tensor: offset + first row * C / 8), and two strips are checked against the oracle."""
    R, C = 8192, 8352
    g = torch.Generator().manual_seed(3)
    f32 = torch.float32
    qx, sx = jf.quantize(torch.randn(R, C, generator=g).cuda(), scale_dtype=f32)
    qg, sg = jf.quantize((1e-3 * torch.randn(R, C, generator=g)).cuda(), jf.ROUND_STOCHASTIC, f32, seed=0, offset=0)
    eps = 5e-5 if approx == 0 else 0.0
    qy, sy = jf.gelu_fwd(qx, sx, approx, eps)
    qd, sd = jf.gelu_bwd(qx, sx, qg, sg, approx, jf.ROUND_STOCHASTIC, seed=6, offset=4)
    for r0 in range(0, R, 512):
        rows, rb = slice(r0, r0 + 512), slice(r0 // QB, (r0 + 512) // QB)
        py, ps = jf.gelu_fwd(qx[rows], sx[rb], approx, eps)
        assert torch.equal(py, qy[rows]) and torch.equal(ps, sy[rb]), f"forward rows {r0}"
        pd, ps = jf.gelu_bwd(qx[rows], sx[rb], qg[rows], sg[rb], approx, jf.ROUND_STOCHASTIC, seed=6, offset=4 + r0 * C // 8)
        assert torch.equal(pd, qd[rows]) and torch.equal(ps, sd[rb]), f"backward rows {r0}"
    for r0 in (0, R - QB):
        rows, rb = slice(r0, r0 + QB), slice(r0 // QB, r0 // QB + 1)
        X, SX, G, SG = (t.cpu().numpy() for t in (qx[rows], sx[rb], qg[rows], sg[rb]))
        wq, ws = oracle.gelu_fwd(X, SX, approx, eps)
        same(qy[rows], wq, f"forward codes rows {r0}")
        same(sy[rb], ws, f"forward scales rows {r0}")
        wq, ws = oracle.gelu_bwd(X, SX, G, SG, approx, True, 6, 4 + r0 * C // 8)
        same(qd[rows], wq, f"backward codes rows {r0}")
        same(sd[rb], ws, f"backward scales rows {r0}")
