"""GPU parity of the memory-bound kernels (quantise, transpose, dequantise, LayerNorm, GELU, add)
against the CPU oracle, through the C ABI.  INT8 codes and scales: bit-exact.  fp32 outputs of
elementwise kernels: bit-exact; reductions that end in fp outputs (dgamma, dbeta): 1e-5 relative.
"""
import numpy as np
import pytest
import torch

from helpers import QB, expand_scales, rand_codes, rand_scales
from test_gpu_gemm import dev, same

pytestmark = pytest.mark.gpu

SHAPES = [(32, 32), (64, 96), (96, 160), (256, 1600)]
ROUND = {"nearest": 0, "stochastic": 1, "trunc": 2, "stochastic_trunc": 3}


def rand_x(rng, R, C):
    x = (rng.standard_normal((R, C)) * np.exp2(rng.integers(-6, 3, (R, C)))).astype(np.float32)
    if R >= 64:
        x[32:64, :32] = 0.0        # an all-zero block
    return x


def block_tensor(oracle, rng, R, C, scale=1.0, f16=True):
    q, s = oracle.quantize((rng.standard_normal((R, C)) * scale).astype(np.float32), scale_dtype="f16" if f16 else "f32")
    return q, s


@pytest.mark.parametrize("f16", [True, False])
@pytest.mark.parametrize("mode", ["nearest", "stochastic", "trunc", "stochastic_trunc"])
@pytest.mark.parametrize("R,C", SHAPES)
def test_quantize(jf, oracle, R, C, mode, f16):
    print(f"case quantize {R}x{C} {mode} f16={f16}", flush=True)
    rng = np.random.default_rng(R + C)
    x = rand_x(rng, R, C)
    sd = torch.float16 if f16 else torch.float32
    q, s = jf.quantize(dev(x), rounding=ROUND[mode], scale_dtype=sd, seed=42, offset=17)
    wq, ws = oracle.quantize(x, stochastic="stochastic" in mode, seed=42, offset=17, truncate="trunc" in mode,
                             scale_dtype="f16" if f16 else "f32")
    same(q, wq, "codes")
    same(s, ws, "scales")


@pytest.mark.parametrize("R,C", [(96, 160), (32, 32), (160, 96), (288, 1056), (1056, 288)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_quantize_half_inputs_and_transpose(jf, oracle, dtype, R, C):
    """(shapes: row-block counts that are not multiples of 4 and column-block counts that are not multiples of 4: the
    kernel's walk with a transposed copy takes quads of row blocks and groups of four column blocks)"""
    rng = np.random.default_rng(3)
    x = torch.from_numpy(rand_x(rng, R, C)).to(dtype)
    q, s, qT = jf.quantize(x.cuda(), rounding=jf.ROUND_STOCHASTIC, transpose=True, seed=5, offset=0)
    wq, ws = oracle.quantize(x.float().numpy(), stochastic=True, seed=5, offset=0, scale_dtype="f16")
    same(q, wq, "codes")
    same(s, ws, "scales")
    same(qT, np.ascontiguousarray(wq.T), "transposed codes")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mode", ["nearest", "stochastic"])
def test_quantize_slabs_equal_the_quantised_concatenation(jf, oracle, dtype, mode):
    """Column slabs quantised where they lie (jf_quantize_slabs: unit column stride, any row stride) give the codes,
    scales and rounding noise of jf_quantize on their concatenation, and of the oracle on it."""
    rng = np.random.default_rng(11)
    R, widths = 96, (64, 160, 32)
    parts = [torch.from_numpy(rand_x(rng, R, w) * (0.2 + i)).to(dtype).cuda() for i, w in enumerate(widths)]
    wide = torch.from_numpy(rand_x(rng, R, 224)).to(dtype).cuda()
    parts[1] = wide[:, 32:192]                                  # a slab with a row stride of its own (224 elements)
    cat = torch.cat(parts, dim=1)
    sd = torch.float16
    q, s = jf.quantize_slabs(parts, ROUND[mode], sd, seed=42, offset=17)
    q0, s0 = jf.quantize(cat, ROUND[mode], sd, seed=42, offset=17)
    assert torch.equal(q, q0) and torch.equal(s, s0)
    wq, ws = oracle.quantize(cat.float().cpu().numpy(), stochastic=mode == "stochastic", seed=42, offset=17, scale_dtype="f16")
    same(q, wq, "codes")
    same(s, ws, "scales")
    with pytest.raises(RuntimeError):
        jf.quantize_slabs([parts[0], parts[1][:64]])            # rows differ
    with pytest.raises(RuntimeError):
        jf.quantize_slabs([parts[0], wide[:, 1:33]])            # a slab that does not start on a 16-byte boundary


def test_quantize_amax_eps_and_tiny_scales(jf, oracle):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((64, 64)) * 1e-25).astype(np.float32)     # scale below the fast-division range
    x[:32, :32] *= 1e-10
    q, s = jf.quantize(dev(x), scale_dtype=torch.float32)
    wq, ws = oracle.quantize(x)
    same(q, wq, "codes")
    same(s, ws, "scales")
    q, s = jf.quantize(dev(x), scale_dtype=torch.float32, amax_eps=5e-5)
    wq, ws = oracle.quantize(x, amax_eps=5e-5)
    same(q, wq, "codes eps")
    same(s, ws, "scales eps")


@pytest.mark.parametrize("R,C", [(32, 32), (96, 160), (16, 48), (48, 80), (80, 16), (208, 1040), (1040, 528), (1600, 8192)])
def test_transpose(jf, R, C):
    rng = np.random.default_rng(R)
    q = rand_codes(rng, (R, C))
    same(jf.transpose_s8(dev(q)), np.ascontiguousarray(q.T), "transpose")


@pytest.mark.parametrize("f16", [True, False])
def test_dequantize(jf, oracle, f16):
    rng = np.random.default_rng(6)
    q = rand_codes(rng, (96, 160))
    s = rand_scales(rng, (3, 5), f16=f16)
    got = jf.dequantize(dev(q), dev(s.astype(np.float16 if f16 else np.float32)))
    same(got, oracle.dequantize(q, s), "dequantize")
    # 16-bit outputs: the fp32 product rounded once (for binary16 scales: the reference's binary16 multiplication)
    want = torch.from_numpy(oracle.dequantize(q, s))
    for dt in (torch.float16, torch.bfloat16):
        got16 = jf.dequantize(dev(q), dev(s.astype(np.float16 if f16 else np.float32)), out_dtype=dt)
        assert got16.dtype == dt and torch.equal(got16.cpu(), want.to(dt)), f"dequantize to {dt}"
    if f16:
        prod = torch.from_numpy(q).to(torch.float16).reshape(q.shape[0] // 32, 32, q.shape[1] // 32, 32) * \
            torch.from_numpy(s.astype(np.float16)).unsqueeze(1).unsqueeze(3)
        assert torch.equal(jf.dequantize(dev(q), dev(s.astype(np.float16)), out_dtype=torch.float16).cpu(),
                           prod.reshape(q.shape)), "binary16 product (linear_fwd.py:29)"


@pytest.mark.parametrize("f16", [True, False])
@pytest.mark.parametrize("approx,eps", [(0, 5e-5), (1, 0.0)])
@pytest.mark.parametrize("R,C", SHAPES)
def test_gelu_fwd_bwd(jf, oracle, R, C, approx, eps, f16):
    print(f"case gelu {R}x{C} approx={approx} f16={f16}", flush=True)
    rng = np.random.default_rng(R * 3 + C + approx)
    st = np.float16 if f16 else np.float32
    sdt = "f16" if f16 else "f32"
    qx, sx = block_tensor(oracle, rng, R, C, 2.0, f16)
    qg, sg = block_tensor(oracle, rng, R, C, 1e-3, f16)
    qy, sy = jf.gelu_fwd(dev(qx), dev(sx), approx, eps)
    wq, ws = oracle.gelu_fwd(qx, sx.astype(np.float32), approx, eps, scale_dtype=sdt)
    same(qy, wq, "fwd codes")
    same(sy, ws, "fwd scales")
    for rounding, stochastic in ((0, False), (1, True)):
        qd, sd = jf.gelu_bwd(dev(qx), dev(sx), dev(qg), dev(sg), approx, rounding, seed=8, offset=3)
        wq, ws = oracle.gelu_bwd(qx, sx.astype(np.float32), qg, sg.astype(np.float32), approx, stochastic, 8, 3,
                                 scale_dtype=sdt)
        same(qd, wq, f"bwd codes stochastic={stochastic}")
        same(sd, ws, "bwd scales")


def test_gelu_fwd_close_to_torch(jf, oracle):
    """1e-3 relative on dequantised outputs vs torch's erf GELU of the dequantised input."""
    rng = np.random.default_rng(12)
    qx, sx = block_tensor(oracle, rng, 256, 512, 1.5, f16=False)   # fp32 scales: the stored scale is the one used
    qy, sy = jf.gelu_fwd(dev(qx), dev(sx))
    y = jf.dequantize(qy, sy).cpu().numpy()
    x = torch.from_numpy(qx * expand_scales(sx.astype(np.float32)).astype(np.float64))
    ref = torch.nn.functional.gelu(x).numpy()
    step = expand_scales(sy.cpu().numpy().astype(np.float32))
    assert np.all(np.abs(y - ref) <= 0.5 * step * (1 + 1e-3) + 1e-3 * np.abs(ref))


@pytest.mark.parametrize("f16", [True, False])
@pytest.mark.parametrize("R,C", SHAPES)
def test_rowstats_layernorm(jf, oracle, R, C, f16):
    print(f"case layernorm {R}x{C} f16={f16}", flush=True)
    rng = np.random.default_rng(R + 7 * C)
    sdt = "f16" if f16 else "f32"
    qx, sx = block_tensor(oracle, rng, R, C, 1.0, f16)
    qg, sg = block_tensor(oracle, rng, R, C, 1e-3, f16)
    gamma = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(C)).astype(np.float32)
    mean, rstd = jf.rowstats(dev(qx), dev(sx), 1e-5)
    wm, wr = oracle.rowstats(qx, sx.astype(np.float32), 1e-5)
    same(mean, wm, "mean")
    same(rstd, wr, "rstd")
    for b in (beta, None):
        qy, sy = jf.layernorm_fwd(dev(qx), dev(sx), dev(gamma), None if b is None else dev(b), mean, rstd)
        wq, ws = oracle.layernorm_fwd(qx, sx.astype(np.float32), gamma, b, wm, wr, scale_dtype=sdt)
        same(qy, wq, "fwd codes")
        same(sy, ws, "fwd scales")
    for rounding, stochastic in ((0, False), (1, True)):
        qd, sd, dg, db = jf.layernorm_bwd(dev(qx), dev(sx), dev(qg), dev(sg), dev(gamma), mean, rstd, rounding,
                                          seed=77, offset=1)
        wq, ws, wdg, wdb = oracle.layernorm_bwd(qx, sx.astype(np.float32), qg, sg.astype(np.float32), gamma, wm, wr,
                                                stochastic, 77, 1, scale_dtype=sdt)
        same(qd, wq, f"bwd codes stochastic={stochastic}")
        same(sd, ws, "bwd scales")
        assert np.allclose(dg.cpu().numpy(), wdg, rtol=1e-5, atol=1e-5 * np.abs(wdg).max())
        assert np.allclose(db.cpu().numpy(), wdb, rtol=1e-5, atol=1e-5 * np.abs(wdb).max())


def test_layernorm_vs_torch(jf, oracle):
    """Against torch.nn.functional.layer_norm + autograd on the dequantised operands."""
    rng = np.random.default_rng(21)
    R, C = 128, 1600
    qx, sx = block_tensor(oracle, rng, R, C, 1.0, f16=False)       # fp32 scales: the stored scale is the one used
    qg, sg = block_tensor(oracle, rng, R, C, 1e-3, f16=False)
    gamma = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(C)).astype(np.float32)
    mean, rstd = jf.rowstats(dev(qx), dev(sx), 1e-5)
    qy, sy = jf.layernorm_fwd(dev(qx), dev(sx), dev(gamma), dev(beta), mean, rstd)
    qd, sd, dg, db = jf.layernorm_bwd(dev(qx), dev(sx), dev(qg), dev(sg), dev(gamma), mean, rstd)
    x = torch.tensor(qx * expand_scales(sx.astype(np.float32)).astype(np.float64), requires_grad=True)
    gt = torch.tensor(gamma.astype(np.float64), requires_grad=True)
    bt = torch.tensor(beta.astype(np.float64), requires_grad=True)
    y = torch.nn.functional.layer_norm(x, (C,), gt, bt, 1e-5)
    y.backward(torch.tensor(qg * expand_scales(sg.astype(np.float32)).astype(np.float64)))
    for (q, s, ref) in ((qy, sy, y.detach().numpy()), (qd, sd, x.grad.numpy())):
        got = jf.dequantize(q, s).cpu().numpy()
        step = expand_scales(s.cpu().numpy().astype(np.float32))
        assert np.all(np.abs(got - ref) <= 0.5 * step * (1 + 2e-3) + 1e-3 * np.abs(ref))
    assert np.allclose(dg.cpu().numpy(), gt.grad.numpy(), rtol=1e-3, atol=1e-6)
    assert np.allclose(db.cpu().numpy(), bt.grad.numpy(), rtol=1e-3, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mode", ["trunc", "nearest", "stochastic_trunc", "stochastic"])
def test_add(jf, oracle, dtype, mode):
    rng = np.random.default_rng(31)
    R, C = 96, 160
    x1 = torch.from_numpy(rng.standard_normal((R, C)).astype(np.float32)).to(dtype)
    q2, s2 = block_tensor(oracle, rng, R, C, 0.5)
    y1, q, s, rs, rq = jf.add(x1.cuda(), dev(q2), dev(s2), ROUND[mode], with_stats=True, seed=9, offset=2)
    wy, wq, ws, wrs, wrq = oracle.add(x1.float().numpy(), q2, s2.astype(np.float32), "stochastic" in mode, 9, 2,
                                      "trunc" in mode, True, "f16")
    same(y1, wy, "fp sum")
    same(q, wq, "codes")
    same(s, ws, "scales")
    same(rs, wrs, "row sums")
    same(rq, wrq, "row square sums")
    # the finishing step: partials added in ascending order, var = E[y^2] - mean^2, rstd = 1/sqrt(var), all in binary32
    mean, rstd = jf.rowstats_finish(rs, rq, C)
    a, b = np.zeros(R, np.float32), np.zeros(R, np.float32)
    for j in range(C // 32):
        a, b = a + wrs[j], b + wrq[j]
    m = a / np.float32(C)
    var = b / np.float32(C) - m * m
    same(mean, m, "mean")
    same(rstd, np.float32(1) / np.sqrt(var), "rstd")
    assert np.allclose(m, wy.mean(-1), atol=1e-5) and np.allclose(rstd.cpu().numpy(), 1 / np.sqrt(wy.var(-1)), rtol=1e-4)


@pytest.mark.parametrize("R,C", [(64, 96), (96, 1600), (32, 2048), (64, 2080)])
@pytest.mark.parametrize("x1_dtype,out_dtype,scale_dtype", [(torch.float32, torch.float32, torch.float32),
                                                            (torch.bfloat16, torch.bfloat16, torch.float16),
                                                            (torch.float16, torch.float32, torch.float16),
                                                            (torch.float32, torch.bfloat16, torch.float32)])
def test_layernorm_backward_with_the_residual_add(jf, R, C, x1_dtype, out_dtype, scale_dtype):
    """One kernel for LayerNorm backward + the residual add that follows it in the recipe (rows of up to 2048 columns;
    2080 columns make the two calls inside the wrapper): the same bits as the two calls, which are checked against the
    CPU checker one by one above."""
    g = torch.Generator().manual_seed(R + C)
    x = torch.randn(R, C, generator=g).cuda()
    dy = (torch.randn(R, C, generator=g) * 1e-2).cuda()
    gamma = (1 + 0.1 * torch.randn(C, generator=g)).cuda()
    x1 = (torch.randn(R, C, generator=g) * 1e-2).to(x1_dtype).cuda()
    qx, sx = jf.quantize(x, scale_dtype=scale_dtype)
    qg, sg = jf.quantize(dy, jf.ROUND_STOCHASTIC, scale_dtype, seed=4, offset=0)
    mean, rstd = jf.rowstats(qx, sx)
    for want_dbeta in (True, False):
        for r1, r2 in ((jf.ROUND_STOCHASTIC, jf.ROUND_STOCHASTIC_TRUNC), (jf.ROUND_NEAREST, jf.ROUND_TRUNC)):
            qdx, sdx, dg, db = jf.layernorm_bwd(qx, sx, qg, sg, gamma, mean, rstd, r1, want_dbeta, seed=7, offset=3)
            wy, wq, ws = jf.add(x1, qdx, sdx, r2, seed=8, offset=5, out_dtype=out_dtype)
            y1, q, s, dg2, db2 = jf.layernorm_bwd_add(qx, sx, qg, sg, gamma, mean, rstd, x1, r1, r2, want_dbeta, out_dtype,
                                                      seed=7, offset=3, add_seed=8, add_offset=5)
            assert y1.dtype == out_dtype and torch.equal(y1, wy)
            assert torch.equal(q, wq) and torch.equal(s, ws)
            assert torch.equal(dg, dg2)
            assert (db is None and db2 is None) or torch.equal(db, db2)
    assert int(q.abs().max()) > 100                                 # a real block tensor came out


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_add_with_a_16_bit_sum(jf, oracle, dtype, out_dtype):
    """The sum may leave the kernel already cast (the reference casts it afterwards, qmodel.py:228): it is the fp32 sum
    rounded to nearest even, and codes, scales and row statistics are those of the fp32 sum."""
    rng = np.random.default_rng(32)
    R, C = 64, 224
    x1 = torch.from_numpy(rng.standard_normal((R, C)).astype(np.float32) * 3).to(dtype)
    q2, s2 = block_tensor(oracle, rng, R, C, 0.5)
    y32, q32, s32, rs32, rq32 = jf.add(x1.cuda(), dev(q2), dev(s2), ROUND["stochastic"], with_stats=True, seed=9, offset=2)
    y16, q, s, rs, rq = jf.add(x1.cuda(), dev(q2), dev(s2), ROUND["stochastic"], with_stats=True, seed=9, offset=2,
                               out_dtype=out_dtype)
    wy, wq, ws, wrs, wrq = oracle.add(x1.float().numpy(), q2, s2.astype(np.float32), True, 9, 2, False, True, "f16")
    assert y16.dtype == out_dtype
    assert torch.equal(y16.cpu(), torch.from_numpy(wy).to(out_dtype))      # torch's cast rounds to nearest even
    assert torch.equal(y16, y32.to(out_dtype))
    same(q, wq, "codes")
    same(s, ws, "scales")
    same(rs, wrs, "row sums")
    same(rq, wrq, "row square sums")
    with pytest.raises(RuntimeError):
        jf.add(x1.cuda(), dev(q2), dev(s2), out_dtype=torch.float64)


def test_full_size_nonlinear_properties(jf, oracle):
    """benchmark configuration 4 sizes.  Checked bit-exactly against the oracle on row slabs (the kernels are
    block-local, so a slab of the input is a complete problem), and by size-independent properties."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(8192, 6400, generator=g)
    qx, sx = jf.quantize(x.cuda(), scale_dtype=torch.float32)
    qy, sy = jf.gelu_fwd(qx, sx, jf.GELU_TANH, 0.0)
    assert int(qy.abs().max()) == 127
    blocks = qy.reshape(256, 32, 200, 32).abs().amax(dim=(1, 3))
    assert bool((blocks == 127).all())                      # every non-zero block uses the full code range
    for r0 in (0, 4096, 8160):
        wq, ws = oracle.gelu_fwd(qx[r0:r0 + 32].cpu().numpy(), sx[r0 // 32:r0 // 32 + 1].cpu().numpy(), 1, 0.0)
        same(qy[r0:r0 + 32], wq, f"gelu codes rows {r0}")
        same(sy[r0 // 32:r0 // 32 + 1], ws, f"gelu scales rows {r0}")
    # quantise(dequantise(q, s)) == (q, s): idempotence at full size
    back = jf.dequantize(qy, sy)
    q2, s2 = jf.quantize(back, scale_dtype=torch.float32)
    assert torch.equal(q2, qy)
    # transpose twice is the identity
    assert torch.equal(jf.transpose_s8(jf.transpose_s8(qy)), qy)


def test_full_size_layernorm_backward_with_the_residual_add(jf, oracle):
    """8192 x 1600, stochastic, binary16 scales, bfloat16 gradient in and out (what a block of the recipe runs): the
    one-kernel form against the two calls at full size, and three strips of the two calls against the CPU checker."""
    R, C = 8192, 1600
    g = torch.Generator().manual_seed(5)
    x = torch.randn(R, C, generator=g).cuda()
    dy = (torch.randn(R, C, generator=g) * 1e-3).cuda()
    gamma = (1 + 0.1 * torch.randn(C, generator=g)).cuda()
    x1 = (torch.randn(R, C, generator=g) * 1e-3).to(torch.bfloat16).cuda()
    qx, sx = jf.quantize(x, scale_dtype=torch.float16)
    qg, sg = jf.quantize(dy, jf.ROUND_STOCHASTIC, torch.float16, seed=1, offset=0)
    mean, rstd = jf.rowstats(qx, sx)
    qdx, sdx, dg, db = jf.layernorm_bwd(qx, sx, qg, sg, gamma, mean, rstd, jf.ROUND_STOCHASTIC, True, seed=2, offset=11)
    wy, wq, ws = jf.add(x1, qdx, sdx, jf.ROUND_STOCHASTIC_TRUNC, seed=3, offset=17, out_dtype=torch.bfloat16)
    y1, q, s, dg2, db2 = jf.layernorm_bwd_add(qx, sx, qg, sg, gamma, mean, rstd, x1, jf.ROUND_STOCHASTIC,
                                              jf.ROUND_STOCHASTIC_TRUNC, True, torch.bfloat16, seed=2, offset=11,
                                              add_seed=3, add_offset=17)
    assert torch.equal(y1, wy) and torch.equal(q, wq) and torch.equal(s, ws)
    assert torch.equal(dg, dg2) and torch.equal(db, db2)
    for r0 in (0, 4096, 8160):
        sl, bl = slice(r0, r0 + 32), slice(r0 // 32, r0 // 32 + 1)
        oy, oq, os_ = oracle.add(x1[sl].float().cpu().numpy(), qdx[sl].cpu().numpy(), sdx[bl].float().cpu().numpy(), True, 3,
                                 17 + r0 * C // 8, True, False, "f16")
        assert torch.equal(y1[sl].cpu(), torch.from_numpy(oy).to(torch.bfloat16)), r0
        same(q[sl], oq, f"codes rows {r0}")
        same(s[bl], os_, f"scales rows {r0}")


def _random_block_shapes(n, seed):
    rng = np.random.default_rng(seed)
    for _ in range(n):
        yield int(rng.integers(1, 11)) * 32, int(rng.integers(1, 130)) * 32, bool(rng.integers(0, 2)), int(rng.integers(0, 2))


@pytest.mark.parametrize("R,C", [(64, 2048), (64, 2080), (32, 1632), (96, 512), (32, 544)])
def test_layernorm_backward_single_pass_and_two_launch_forms(jf, oracle, R, C):
    """Rows of up to 64 column blocks (2048 columns) take the single-pass strip kernel, wider rows the two-launch form:
    the widest row of the first, the narrowest of the second, rows whose block count is not a multiple of the 16 waves
    of a strip, and rows of exactly / just over 16 blocks."""
    test_rowstats_layernorm(jf, oracle, R, C, False)
    test_rowstats_layernorm(jf, oracle, R, C, True)


@pytest.mark.parametrize("R,C,f16,approx", list(_random_block_shapes(12, 7)))
def test_random_shapes(jf, oracle, R, C, f16, approx):
    """The GELU and LayerNorm checks above on random tensor shapes (up to 320 x 4128: rows of more column blocks than a
    workgroup has waves, block counts that are not multiples of the grid)."""
    test_gelu_fwd_bwd(jf, oracle, R, C, approx, 5e-5 if approx == 0 else 0.0, f16)
    test_rowstats_layernorm(jf, oracle, R, C, f16)
    test_quantize(jf, oracle, R, C, "stochastic", f16)


@pytest.mark.parametrize("R,C", [(32, 32), (96, 160), (2080, 288), (8192 + 64, 1600), (12288, 768)])
@pytest.mark.parametrize("f16", [True, False])
def test_block_column_sums(jf, oracle, R, C, f16):
    """jf_block_colsum (the bias gradient) against the oracle's restatement of its summation order, bit for bit; shapes
    with fewer strips than partial sums, strip counts that are not multiples of 32 or 256, widths that are not multiples
    of the 256 columns a wave takes."""
    rng = np.random.default_rng(R + C)
    q = rand_codes(rng, (R, C), sparse=0.1)
    s = rand_scales(rng, (R // QB, C // QB), f16=f16)
    ds = torch.from_numpy(s).cuda()
    got = jf.block_colsum(torch.from_numpy(q).cuda(), ds.half() if f16 else ds)
    want = oracle.block_colsum(q, s)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("approx,eps", [(0, 5e-5), (1, 0.0), (0, 0.0)])
@pytest.mark.parametrize("f16", [True, False])
def test_gelu_fwd_on_one_sided_and_degenerate_blocks(jf, oracle, approx, eps, f16):
    """Blocks whose absmax is not where random data puts it: only negative codes, on one side of the minimum of x*Phi(x)
    (at x = -0.75) or straddling it, a single code, the byte -128, far tails where the outputs are a few units of 2^-24,
    all zeros, a zero scale, scales from 1e-4 to 40; blocks whose largest positive output lies just below or above the
    largest magnitude a negative input can produce."""
    rng = np.random.default_rng(77 + approx)
    blocks, scales = [], []

    def add(codes, scale):
        b = np.asarray(codes, dtype=np.int8)
        blocks.append(np.resize(b, (QB, QB)) if b.size != QB * QB else b.reshape(QB, QB))
        scales.append(scale)
    for scale in (0.0059, 0.01, 0.0387, 0.1, 0.75, 3.0, 1e-4, 40.0):
        ks = min(int(0.7518 / scale), 127)
        add(rng.integers(-127, 0, QB * QB), scale)                           # negative only
        add(rng.integers(-max(ks, 1), 1, QB * QB), scale)                    # up to the split
        add(rng.integers(-127, -min(ks + 1, 127) + 1, QB * QB), scale)       # beyond the split
        add([-min(ks, 127) or -1, -min(ks + 1, 127)], scale)                 # the two codes around the minimum
        add([-127, -124], scale)                                             # two far-tail codes
        add([-128, -127, 5], scale)                                          # the byte -128
        add([int(rng.integers(-127, 128))], scale)                           # one code
        add(rng.integers(-127, 128, QB * QB), scale)
        add(np.where(rng.random(QB * QB) < 0.9, 0, rng.integers(-127, 0, QB * QB)), scale)
        # the largest positive output on either side of 0.1701 (x = 0.279), where the kernel changes how it finds the
        # block's absmax, with negative codes on both sides of the minimum; one positive element among negative ones
        kp = min(int(0.279 / scale), 126)
        for top in (kp, kp + 1):
            if top >= 1:
                add(np.where(rng.random(QB * QB) < 0.5, rng.integers(1, top + 1, QB * QB), rng.integers(-127, 0, QB * QB)), scale)
        lone = rng.integers(-127, 0, QB * QB)
        lone[int(rng.integers(0, QB * QB))] = int(rng.integers(1, 128))
        add(lone, scale)
    add(np.zeros(QB * QB), 1.0)
    add(rng.integers(-127, 128, QB * QB), 0.0)
    n = len(blocks)
    cols = 8
    rows = -(-n // cols)
    while len(blocks) < rows * cols:
        add(rng.integers(-127, 128, QB * QB), 0.5)
    q = np.block([[blocks[r * cols + c] for c in range(cols)] for r in range(rows)])
    s = np.array(scales, np.float32).reshape(rows, cols)
    if f16:
        s = s.astype(np.float16).astype(np.float32)
    ds = torch.from_numpy(s).cuda()
    qy, sy = jf.gelu_fwd(torch.from_numpy(q).cuda(), ds.half() if f16 else ds, approx, eps)
    wq, ws = oracle.gelu_fwd(q, s, approx, eps, scale_dtype="f16" if f16 else "f32")
    same(sy, ws, "scales")
    same(qy, wq, "codes")
