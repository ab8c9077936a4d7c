"""GPU parity of the per-block INT8 GEMMs (through the C ABI) against the CPU oracle.

Bars: INT32 results, per-K-block INT32 accumulators, INT8 codes and scales: bit-exact.  The fp32
accumulation is compared bit-exact too (same fmaf chain); fp16 output = RNE of it.
Shapes: the reference's own test lists (JetfireGEMMKernel/tests/*.py) plus shapes that are not
multiples of the 128x128 tile (where the reference drops tiles) and a K with an odd number of blocks.
"""
import os

import numpy as np
import pytest
import torch

from helpers import QB, rand_codes, rand_scales

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden")
SHAPES = [(128, 256, 32), (512, 512, 64), (32, 32, 32), (96, 160, 224), (160, 96, 96), (256, 384, 544)]


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def same(got, want, what):
    got = got.cpu().numpy() if isinstance(got, torch.Tensor) else got
    if got.dtype == np.float16:
        g, w = got.view(np.uint16), want.view(np.uint16)
    elif got.dtype == np.float32:
        g, w = got.view(np.uint32), want.view(np.uint32)
    else:
        g, w = got, want
    bad = np.argwhere(g != w)
    assert bad.shape[0] == 0, f"{what}: {bad.shape[0]} of {g.size} differ; first at {bad[0].tolist()}: " \
                              f"got {got[tuple(bad[0])]}, want {want[tuple(bad[0])]}"


def make_problem(seed, M, N, K, f16=True):
    rng = np.random.default_rng(seed)
    A = rand_codes(rng, (M, K))
    Bkn = rand_codes(rng, (K, N))
    sa = rand_scales(rng, (K // QB, M // QB), f16=f16)
    sb = rand_scales(rng, (K // QB, N // QB), f16=f16)
    return A, Bkn, sa, sb


def b_of(Bkn, layout):
    return Bkn if layout == 1 else np.ascontiguousarray(Bkn.T)


def test_reference_fixture(jf, oracle):
    """A/B/CPU dump of the reference's igemm_BasicInt8Gemm_128_128_32 harness."""
    A = np.loadtxt(os.path.join(GOLD, "basic_int8_gemm_128_128_32_A.txt"), dtype=np.int64).reshape(128, 32).astype(np.int8)
    B = np.loadtxt(os.path.join(GOLD, "basic_int8_gemm_128_128_32_B.txt"), dtype=np.int64).reshape(32, 128).astype(np.int8)
    Cw = np.loadtxt(os.path.join(GOLD, "basic_int8_gemm_128_128_32_C.txt"), dtype=np.int64).reshape(128, 128).astype(np.int32)
    same(jf.igemm_s32(dev(A), dev(B), jf.B_KN), Cw, "fixture KN")
    same(jf.igemm_s32(dev(A), dev(np.ascontiguousarray(B.T)), jf.B_NK), Cw, "fixture NK")


@pytest.mark.parametrize("layout", [0, 1])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_s32_and_block_accumulators(jf, oracle, M, N, K, layout):
    print(f"case s32 M={M} N={N} K={K} layout={layout}", flush=True)
    A, Bkn, _, _ = make_problem(M * 7 + N * 3 + K, M, N, K)
    B = b_of(Bkn, layout)
    same(jf.igemm_s32(dev(A), dev(B), layout), oracle.igemm_s32(A, B, layout), "s32")
    same(jf.igemm_block_acc(dev(A), dev(B), layout), oracle.igemm_block_acc(A, B, layout), "block acc")


def test_s32_extreme_codes(jf):
    A = np.full((64, 96), -127, np.int8)
    B = np.full((96, 64), 127, np.int8)
    got = jf.igemm_s32(dev(A), dev(B), jf.B_KN).cpu().numpy()
    assert np.all(got == -96 * 127 * 127)


@pytest.mark.parametrize("f16", [True, False])
@pytest.mark.parametrize("layout", [0, 1])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_block_fp(jf, oracle, M, N, K, layout, f16):
    print(f"case fp M={M} N={N} K={K} layout={layout} f16={f16}", flush=True)
    A, Bkn, sa, sb = make_problem(M + N + K + layout, M, N, K, f16)
    B = b_of(Bkn, layout)
    st = np.float16 if f16 else np.float32
    want32 = oracle.igemm_block_f32(A, B, sa, sb, layout)
    got32 = jf.igemm_block_fp(dev(A), dev(B), dev(sa.astype(st)), dev(sb.astype(st)), layout, torch.float32)
    same(got32, want32, "fp32 accumulators")
    got16 = jf.igemm_block_fp(dev(A), dev(B), dev(sa.astype(st)), dev(sb.astype(st)), layout, torch.float16)
    with np.errstate(over="ignore"):
        same(got16, want32.astype(np.float16), "fp16 output")
    gotbf = jf.igemm_block_fp(dev(A), dev(B), dev(sa.astype(st)), dev(sb.astype(st)), layout, torch.bfloat16)
    wantbf = torch.from_numpy(want32).to(torch.bfloat16)
    assert torch.equal(gotbf.cpu(), wantbf)


@pytest.mark.parametrize("f16", [True, False])
@pytest.mark.parametrize("layout", [0, 1])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_block_q_deterministic_and_stochastic(jf, oracle, M, N, K, layout, f16):
    print(f"case q M={M} N={N} K={K} layout={layout} f16={f16}", flush=True)
    A, Bkn, sa, sb = make_problem(M * 3 + N + K + layout, M, N, K, f16)
    B = b_of(Bkn, layout)
    st = np.float16 if f16 else np.float32
    sdt = "f16" if f16 else "f32"
    dA, dB, dsa, dsb = dev(A), dev(B), dev(sa.astype(st)), dev(sb.astype(st))
    q, sc = jf.igemm_block_q(dA, dB, dsa, dsb, layout)
    wq, wsc = oracle.igemm_block_q(A, B, sa, sb, layout, scale_dtype=sdt)
    same(q, wq, "det codes")
    same(sc, wsc, "det scales")
    q2, sc2 = jf.igemm_block_q(dA, dB, dsa, dsb, layout)
    assert torch.equal(q, q2) and torch.equal(sc, sc2), "run-to-run difference"
    for seed, offset in ((0, 0), (0x1234567890ABCDEF, 977)):
        q, sc = jf.igemm_block_q(dA, dB, dsa, dsb, layout, rounding=jf.ROUND_STOCHASTIC, seed=seed, offset=offset)
        wq, wsc = oracle.igemm_block_q(A, B, sa, sb, layout, stochastic=True, seed=seed, offset=offset, scale_dtype=sdt)
        same(q, wq, f"SR codes seed={seed}")
        same(sc, wsc, "SR scales")


@pytest.mark.parametrize("f16", [True, False])
@pytest.mark.parametrize("layout", [0, 1])
def test_row_major_scale_operands(jf, oracle, layout, f16):
    """The scale operands may be the .t() views of the block tensors' own [rows/32, K/32] scale arrays (no transposed
    copy): same bits as with K-major copies, for each operand separately and for both."""
    M, N, K = 160, 352, 544
    A, Bkn, sa, sb = make_problem(99 + layout, M, N, K, f16)
    B = b_of(Bkn, layout)
    st = np.float16 if f16 else np.float32
    dA, dB = dev(A), dev(B)
    ka, kb = dev(sa.astype(st)), dev(sb.astype(st))                                  # [K/32, rows/32] contiguous
    ra, rb = dev(np.ascontiguousarray(sa.astype(st).T)).t(), dev(np.ascontiguousarray(sb.astype(st).T)).t()   # views
    assert not ra.is_contiguous() and not rb.is_contiguous()
    want = oracle.igemm_block_f32(A, B, sa, sb, layout)
    for xa, xb in ((ra, kb), (ka, rb), (ra, rb)):
        same(jf.igemm_block_fp(dA, dB, xa, xb, layout, torch.float32), want, "fp32 accumulators")
        q0, s0 = jf.igemm_block_q(dA, dB, ka, kb, layout, rounding=jf.ROUND_STOCHASTIC, seed=3, offset=5)
        q1, s1 = jf.igemm_block_q(dA, dB, xa, xb, layout, rounding=jf.ROUND_STOCHASTIC, seed=3, offset=5)
        assert torch.equal(q0, q1) and torch.equal(s0, s1)
    with pytest.raises(RuntimeError):
        jf.igemm_block_fp(dA, dB, ka[:, ::2].repeat_interleave(2, 1)[:, : M // QB].t().t()[::1].as_strided((K // QB, M // QB), (M // QB * 2, 2)), kb, layout)


@pytest.mark.parametrize("layout", [0, 1])
@pytest.mark.parametrize("regime", ["huge_everywhere", "huge_one_block", "huge_last_kblock", "denormal_products"])
def test_extreme_scale_products(jf, oracle, regime, layout):
    """Scale products at the ends of the fp32 range.  sa*sb >= 2^102 is where the kernel's pre-scaled factor
    (sa*sb*2^26) overflows and the wave must fall back to the plain conversion; products in the denormal range
    must keep their (reduced) precision.  Results are finite in every regime, and bit-exact like everywhere else."""
    M, N, K = 160, 288, 160
    A, Bkn, sa, sb = make_problem(1234 + layout, M, N, K, f16=False)
    B = b_of(Bkn, layout)
    sa = (sa / sa.max()).astype(np.float32)
    sb = (sb / sb.max()).astype(np.float32)                      # all in (0, 1]
    if regime == "huge_everywhere":
        sa, sb = sa * np.float32(2.0 ** 53), sb * np.float32(2.0 ** 52)
    elif regime == "huge_one_block":                             # one output block (one wave) takes the fallback
        sa[:, 2] *= np.float32(2.0 ** 53)
        sb[:, 5] *= np.float32(2.0 ** 52)
    elif regime == "huge_last_kblock":
        sa[-1, :] *= np.float32(2.0 ** 53)
        sb[-1, :] *= np.float32(2.0 ** 52)
    else:
        sa, sb = sa * np.float32(2.0 ** -70), sb * np.float32(2.0 ** -70)
    want = oracle.igemm_block_f32(A, B, sa, sb, layout)
    assert np.isfinite(want).all() and np.abs(want).max() > 0
    dA, dB, dsa, dsb = dev(A), dev(B), dev(sa), dev(sb)
    same(jf.igemm_block_fp(dA, dB, dsa, dsb, layout, torch.float32), want, f"{regime}: fp32 accumulators")
    q, sc = jf.igemm_block_q(dA, dB, dsa, dsb, layout)
    wq, wsc = oracle.igemm_block_q(A, B, sa, sb, layout, scale_dtype="f32")
    same(q, wq, f"{regime}: codes")
    same(sc, wsc, f"{regime}: scales")


@pytest.mark.parametrize("f16", [True, False])
@pytest.mark.parametrize("M,N,K", SHAPES + [(160, 288, 1056)])
def test_block_fp_a_given_as_km(jf, oracle, M, N, K, f16):
    """Weight-gradient form with the A operand as it lies in memory ([K, M], e.g. the gradient [tokens, C_out]) and
    B as [K, N]: the same bits as with a materialised transpose."""
    print(f"case fp A_KM M={M} N={N} K={K} f16={f16}", flush=True)
    A, Bkn, sa, sb = make_problem(M + 2 * N + K, M, N, K, f16)
    st = np.float16 if f16 else np.float32
    Akm = np.ascontiguousarray(A.T)
    want32 = oracle.igemm_block_f32(A, Bkn, sa, sb, 1)
    dsa, dsb = dev(sa.astype(st)), dev(sb.astype(st))
    same(jf.igemm_block_fp(dev(Akm), dev(Bkn), dsa, dsb, jf.B_KN, torch.float32, a_layout=jf.A_KM), want32, "fp32 accumulators")
    got16 = jf.igemm_block_fp(dev(Akm), dev(Bkn), dsa, dsb, jf.B_KN, torch.float16, a_layout=jf.A_KM)
    with np.errstate(over="ignore"):
        same(got16, want32.astype(np.float16), "fp16 output")
    with pytest.raises(RuntimeError, match="not implemented"):
        jf.igemm_block_fp(dev(Akm), dev(np.ascontiguousarray(Bkn.T)), dsa, dsb, jf.B_NK, torch.float32, a_layout=jf.A_KM)


@pytest.mark.parametrize("a_km", [False, True])
@pytest.mark.parametrize("M,N,K,req", [(128, 256, 2048, 2), (160, 96, 3104, 4), (96, 160, 2560, 0), (64, 64, 12288, 0),
                                           (128, 128, 512, 3), (32, 32, 992, 2), (256, 384, 544, 0)])
def test_block_fp_split_k(jf, oracle, M, N, K, req, a_km):
    """K cut into ordered partial chains: bit-exact against the oracle's composition with the same plan; request 1
    stays the reference arithmetic; the two differ by fp32 rounding only."""
    print(f"case fp splitk M={M} N={N} K={K} request={req} a_km={a_km}", flush=True)
    A, Bkn, sa, sb = make_problem(M + N + K + req, M, N, K, f16=False)
    parts, per = jf.splitk_plan(M, N, K, req)
    assert parts >= 1 and per % 4 == 0 and (parts - 1) * per < K // QB <= parts * per
    if req == 0:
        assert parts > 1 or K // QB < 32 or 2 * ((M + 127) // 128) * ((N + 127) // 128) > 512
    dA = dev(np.ascontiguousarray(A.T)) if a_km else dev(A)
    kw = dict(a_layout=jf.A_KM if a_km else jf.A_MK)
    dsa, dsb = dev(sa), dev(sb)
    want = oracle.igemm_block_f32_splitk(A, Bkn, sa, sb, 1, parts, per)
    one = oracle.igemm_block_f32(A, Bkn, sa, sb, 1)
    got = jf.igemm_block_fp(dA, dev(Bkn), dsa, dsb, jf.B_KN, torch.float32, splitk=req, **kw)
    same(got, want, f"fp32, {parts} parts of {per} K blocks")
    same(jf.igemm_block_fp(dA, dev(Bkn), dsa, dsb, jf.B_KN, torch.float32, splitk=1, **kw), one, "one chain")
    np.testing.assert_allclose(want, one, rtol=1e-5, atol=1e-5 * np.abs(one).max())
    got16 = jf.igemm_block_fp(dA, dev(Bkn), dsa, dsb, jf.B_KN, torch.float16, splitk=req, **kw)
    with np.errstate(over="ignore"):
        same(got16, want.astype(np.float16), "fp16 output")
    if not a_km:                                                  # B as [N,K] takes the same path
        same(jf.igemm_block_fp(dA, dev(np.ascontiguousarray(Bkn.T)), dsa, dsb, jf.B_NK, torch.float32, splitk=req),
             oracle.igemm_block_f32_splitk(A, np.ascontiguousarray(Bkn.T), sa, sb, 0, parts, per), "B as [N,K]")


def _random_cases(n, seed):
    rng = np.random.default_rng(seed)
    for _ in range(n):
        yield (int(rng.integers(1, 13)) * 32, int(rng.integers(1, 13)) * 32, int(rng.integers(1, 41)) * 32,
               int(rng.integers(0, 2)), bool(rng.integers(0, 2)), int(rng.integers(0, 4)), int(rng.integers(0, 1 << 30)))


@pytest.mark.parametrize("M,N,K,layout,f16,scale_views,seed", list(_random_cases(32, 2024)))
def test_random_shapes(jf, oracle, M, N, K, layout, f16, scale_views, seed):
    """Random small problems (M, N up to 384, K up to 1280, all multiples of 32): every output kind, both B layouts, both
    scale dtypes, K-major copies or row-major views of the scales, the [K,M] form of A where it applies."""
    print(f"case random M={M} N={N} K={K} layout={layout} f16={f16} views={scale_views} seed={seed}", flush=True)
    A, Bkn, sa, sb = make_problem(seed, M, N, K, f16)
    B = b_of(Bkn, layout)
    st = np.float16 if f16 else np.float32
    sdt = "f16" if f16 else "f32"
    dA, dB = dev(A), dev(B)
    dsa = dev(np.ascontiguousarray(sa.astype(st).T)).t() if scale_views & 1 else dev(sa.astype(st))
    dsb = dev(np.ascontiguousarray(sb.astype(st).T)).t() if scale_views & 2 else dev(sb.astype(st))
    same(jf.igemm_s32(dA, dB, layout), oracle.igemm_s32(A, B, layout), "s32")
    acc = oracle.igemm_block_f32(A, B, sa, sb, layout)
    same(jf.igemm_block_fp(dA, dB, dsa, dsb, layout, torch.float32), acc, "fp32")
    q, sc = jf.igemm_block_q(dA, dB, dsa, dsb, layout)
    wq, wsc = oracle.requant(acc, scale_dtype=sdt)
    same(q, wq, "det codes")
    same(sc, wsc, "det scales")
    q, sc = jf.igemm_block_q(dA, dB, dsa, dsb, layout, rounding=jf.ROUND_STOCHASTIC, seed=seed, offset=seed % 1000)
    wq, wsc = oracle.requant(acc, stochastic=True, seed=seed, offset=seed % 1000, scale_dtype=sdt)
    same(q, wq, "SR codes")
    same(sc, wsc, "SR scales")
    if layout == 1:
        same(jf.igemm_block_fp(dev(np.ascontiguousarray(A.T)), dB, dsa, dsb, layout, torch.float32, a_layout=jf.A_KM), acc, "fp32, A as [K,M]")
        parts, per = jf.splitk_plan(M, N, K, 0)
        same(jf.igemm_block_fp(dA, dB, dsa, dsb, layout, torch.float32, splitk=0),
             oracle.igemm_block_f32_splitk(A, B, sa, sb, layout, parts, per), f"fp32, {parts} parts")


@pytest.mark.parametrize("views", [0, 3])
@pytest.mark.parametrize("a_km", [False, True])
def test_block_fp_split_k_binary16_scales(jf, oracle, a_km, views):
    """The K split with binary16 scales (fetched as 32-bit words, half selected by index parity) in both scale layouts."""
    M, N, K, req = 96, 160, 4128, 3
    A, Bkn, sa, sb = make_problem(77, M, N, K, f16=True)
    parts, per = jf.splitk_plan(M, N, K, req)
    assert parts == 3
    dA = dev(np.ascontiguousarray(A.T)) if a_km else dev(A)
    h = np.float16
    dsa = dev(np.ascontiguousarray(sa.astype(h).T)).t() if views & 1 else dev(sa.astype(h))
    dsb = dev(np.ascontiguousarray(sb.astype(h).T)).t() if views & 2 else dev(sb.astype(h))
    want = oracle.igemm_block_f32_splitk(A, Bkn, sa, sb, 1, parts, per)
    got = jf.igemm_block_fp(dA, dev(Bkn), dsa, dsb, jf.B_KN, torch.float32, splitk=req, a_layout=jf.A_KM if a_km else jf.A_MK)
    same(got, want, "fp32")


def test_block_q_bias(jf, oracle):
    """The forward kernel's bias / biasmax inputs (…BiasRowCol.cu:313,341,357)."""
    M, N, K = 128, 256, 96
    A, Bkn, sa, sb = make_problem(5, M, N, K)
    B = b_of(Bkn, 0)
    rng = np.random.default_rng(6)
    acc = oracle.igemm_block_f32(A, B, sa, sb, 0)
    bias = (np.abs(acc).mean() * rng.standard_normal(N)).astype(np.float32)
    biasmax = np.array([np.abs(bias).max()], np.float32)
    q, sc = jf.igemm_block_q(dev(A), dev(B), dev(sa.astype(np.float16)), dev(sb.astype(np.float16)), 0,
                             bias=dev(bias), biasmax=dev(biasmax))
    wq, wsc = oracle.igemm_block_q(A, B, sa, sb, 0, bias=bias, biasmax=float(biasmax[0]), scale_dtype="f16")
    same(q, wq, "bias codes")
    same(sc, wsc, "bias scales")


def test_zero_blocks_and_zero_scales(jf, oracle):
    M, N, K = 64, 64, 64
    A, Bkn, sa, sb = make_problem(9, M, N, K)
    A[:32] = 0
    sb[:, 1] = 0.0
    q, sc = jf.igemm_block_q(dev(A), dev(Bkn), dev(sa.astype(np.float16)), dev(sb.astype(np.float16)), 1)
    wq, wsc = oracle.igemm_block_q(A, Bkn, sa, sb, 1, scale_dtype="f16")
    same(q, wq, "codes")
    same(sc, wsc, "scales")
    assert not q.cpu().numpy()[:32].any() and not sc.cpu().numpy()[0].any()


def test_sr_mean_converges(jf, oracle):
    """Mean of R stochastic runs -> un-rounded product, error ~ R^-1/2
    (JetfireGEMMKernel/tests/test_int8igemmoutputIntQuantizeStochastic.py:70-120)."""
    M, N, K = 128, 128, 64
    A, Bkn, sa, sb = make_problem(11, M, N, K)
    dA, dB, dsa, dsb = dev(A), dev(Bkn), dev(sa.astype(np.float16)), dev(sb.astype(np.float16))
    acc = oracle.igemm_block_f32(A, Bkn, sa, sb, 1)
    amax = np.abs(acc.reshape(M // QB, QB, N // QB, QB)).max(axis=(1, 3))
    t = 127.0 * acc / np.repeat(np.repeat(amax, QB, 0), QB, 1)
    errs = []
    for R in (16, 256):
        m = torch.zeros((M, N), dtype=torch.float64, device="cuda")
        for r in range(R):
            q, _ = jf.igemm_block_q(dA, dB, dsa, dsb, 1, rounding=jf.ROUND_STOCHASTIC, seed=3, offset=r * (M * N // 8))
            m += q
        errs.append(float(np.sqrt(np.mean((m.cpu().numpy() / R - t) ** 2))))
    assert errs[0] < 0.5 / 4 and errs[1] < 0.5 / 16 and 2.5 < errs[0] / errs[1] < 6.5


def test_full_size_small_wgrad_deep_k(jf, oracle):
    """benchmark configuration 2 (GPT-2 small, 12288 tokens): the weight gradient of the qkv layer, K = 12288 deep with few
    output tiles (2304 x 768), both operands read in place from their token-major arrays' natural layouts."""
    T, Cin, Cout = 12288, 768, 2304
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, Cin, generator=g)
    dy = torch.randn(T, Cout, generator=g) * 1e-3
    qx, sx = jf.quantize(x.cuda(), scale_dtype=torch.float32)
    qg, sg, qgT = jf.quantize(dy.cuda(), rounding=jf.ROUND_STOCHASTIC, scale_dtype=torch.float32, transpose=True, seed=0, offset=0)
    dw = jf.igemm_block_fp(qgT, qx, sg, sx, jf.B_KN, torch.float32)
    torch.cuda.synchronize()
    GT, X, SG, SX = (t.cpu().numpy() for t in (qgT, qx, sg, sx))
    for r0 in (0, 1120, 2272):
        rows, rb = slice(r0, r0 + 32), slice(r0 // 32, r0 // 32 + 1)
        want = oracle.igemm_block_f32(GT[rows], X, np.ascontiguousarray(SG[:, rb]), SX, 1)
        same(dw[rows], want, f"wgrad rows {r0}")


def test_gemm_entry_points_can_be_captured_in_a_graph(jf, oracle):
    """The GEMM entry points only launch kernels (no allocation, no synchronisation, no memset), so a caller can record
    them into a HIP graph: three replays, with eager work and synchronisations in between, all give the eager result."""
    M, N, K = 256, 384, 2048
    A, Bkn, sa, sb = make_problem(5, M, N, K, f16=False)
    dA, dB, dsa, dsb = dev(A), dev(Bkn), dev(sa), dev(sb)
    L = jf.lib()
    nb = L.jf_igemm_block_fp_workspace_bytes(M, N, K, jf.B_KN, 4)
    assert nb > 0
    ws = torch.empty(nb, dtype=torch.int8, device="cuda")
    q = torch.empty((M, N), dtype=torch.int8, device="cuda")
    sc = torch.empty((M // QB, N // QB), dtype=torch.float32, device="cuda")
    w = torch.empty((M, N), dtype=torch.float32, device="cuda")

    def launch(stream):
        jf.check(L.jf_igemm_block_q(dA.data_ptr(), dB.data_ptr(), dsa.data_ptr(), dsb.data_ptr(), None, None, q.data_ptr(),
                                    sc.data_ptr(), M, N, K, jf.B_KN, 1, 0, 0, jf.ROUND_STOCHASTIC, 9, 4, None, 0, stream))
        jf.check(L.jf_igemm_block_fp(dA.data_ptr(), dB.data_ptr(), dsa.data_ptr(), dsb.data_ptr(), w.data_ptr(), M, N, K,
                                     jf.A_MK, jf.B_KN, 1, 0, 0, 1, 4, ws.data_ptr(), nb, stream))

    launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    eq, esc, ew = q.clone(), sc.clone(), w.clone()
    parts, per = jf.splitk_plan(M, N, K, 4)
    same(ew, oracle.igemm_block_f32_splitk(A, Bkn, sa, sb, 1, parts, per), "eager split-K")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch(torch.cuda.current_stream().cuda_stream)
    for _ in range(3):
        q.zero_(); sc.zero_(); w.zero_(); ws.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(q, eq) and torch.equal(sc, esc) and torch.equal(w, ew)


@pytest.mark.parametrize("approx", [0, 1])
@pytest.mark.parametrize("f16", [True, False])
@pytest.mark.parametrize("M,N,K", [(128, 256, 96), (96, 160, 224), (256, 384, 544), (32, 32, 32)])
def test_forward_gemm_with_fused_gelu(jf, oracle, M, N, K, f16, approx):
    """The fused entry point returns, bit for bit, what the GEMM and then the GELU kernel return (both of which are
    checked against the oracle elsewhere and here)."""
    print(f"case q+gelu M={M} N={N} K={K} f16={f16} approx={approx}", flush=True)
    A, Bkn, sa, sb = make_problem(M + N * 5 + K, M, N, K, f16)
    sa = sa * np.float32(0.05)                                    # outputs of a few units: the interesting range of GELU
    B = b_of(Bkn, 0)
    st = np.float16 if f16 else np.float32
    sa = sa.astype(st).astype(np.float32)
    sdt = "f16" if f16 else "f32"
    dA, dB, dsa, dsb = dev(A), dev(B), dev(sa.astype(st)), dev(sb.astype(st))
    eps = 5e-5 if approx == 0 else 0.0
    q, s, qg, sg = jf.igemm_block_q_gelu(dA, dB, dsa, dsb, approx, eps)
    q0, s0 = jf.igemm_block_q(dA, dB, dsa, dsb, jf.B_NK)
    qg0, sg0 = jf.gelu_fwd(q0, s0, approx, eps)
    assert torch.equal(q, q0) and torch.equal(s, s0) and torch.equal(qg, qg0) and torch.equal(sg, sg0)
    wq, ws = oracle.igemm_block_q(A, B, sa, sb, 0, scale_dtype=sdt)
    wg, wgs = oracle.gelu_fwd(wq, ws.astype(np.float32), approx, eps, scale_dtype=sdt)
    same(q, wq, "codes")
    same(s, ws, "scales")
    same(qg, wg, "gelu codes")
    same(sg, wgs, "gelu scales")
    assert qg.cpu().numpy().any()


@pytest.mark.parametrize("approx", [0, 1])
@pytest.mark.parametrize("f16", [True, False])
@pytest.mark.parametrize("M,N,K", [(128, 256, 96), (96, 160, 224), (256, 384, 544), (32, 32, 32)])
def test_dgrad_gemm_with_fused_gelu_backward(jf, oracle, M, N, K, f16, approx):
    """The fused entry point returns, bit for bit, what the stochastic activation-gradient GEMM and then the GELU
    backward kernel return (with the same two noise streams), and what the oracle computes for that sequence."""
    print(f"case dgrad+gelu_bwd M={M} N={N} K={K} f16={f16} approx={approx}", flush=True)
    A, Bkn, sa, sb = make_problem(M * 2 + N + K * 3, M, N, K, f16)
    rng = np.random.default_rng(M + N + K)
    st = np.float16 if f16 else np.float32
    sdt = "f16" if f16 else "f32"
    xq = rand_codes(rng, (M, N))
    xs = (rand_scales(rng, (M // QB, N // QB), lo=-6, hi=-4, f16=f16)).astype(np.float32)    # pre-activations of a few units
    dA, dB, dsa, dsb, dxq, dxs = dev(A), dev(Bkn), dev(sa.astype(st)), dev(sb.astype(st)), dev(xq), dev(xs.astype(st))
    for rounding2, stochastic2 in ((jf.ROUND_STOCHASTIC, True), (jf.ROUND_NEAREST, False)):
        q, s = jf.igemm_block_q_gelu_bwd(dA, dB, dsa, dsb, dxq, dxs, approx, rounding2, seed=11, offset=3, gelu_seed=12, gelu_offset=40)
        q0, s0 = jf.igemm_block_q(dA, dB, dsa, dsb, jf.B_KN, rounding=jf.ROUND_STOCHASTIC, seed=11, offset=3)
        q1, s1 = jf.gelu_bwd(dxq, dxs, q0, s0, approx, rounding2, seed=12, offset=40)
        assert torch.equal(q, q1) and torch.equal(s, s1)
        wq, ws = oracle.igemm_block_q(A, Bkn, sa, sb, 1, stochastic=True, seed=11, offset=3, scale_dtype=sdt)
        wg, wgs = oracle.gelu_bwd(xq, xs, wq, ws.astype(np.float32), approx, stochastic2, 12, 40, scale_dtype=sdt)
        same(q, wg, "codes")
        same(s, wgs, "scales")
        assert q.cpu().numpy().any()
    with pytest.raises(RuntimeError):
        jf.igemm_block_q_gelu_bwd(dA, dB, dsa, dsb, dxq[:, : N // 2].contiguous(), dxs[:, : N // 64].contiguous(), approx)


@pytest.mark.parametrize("f16", [True, False])
@pytest.mark.parametrize("layout", [0, 1])
@pytest.mark.parametrize("M,N,K", [(128, 256, 96), (96, 160, 224), (256, 384, 544), (32, 32, 32), (160, 1632, 64)])
def test_gemm_with_fused_dequantisation(jf, oracle, M, N, K, layout, f16):
    """jf_igemm_block_q_dequant returns, bit for bit, the dequantisation of what jf_igemm_block_q stores (both roundings,
    every output type), and the oracle's requantised result times its stored scale."""
    print(f"case q+dequant M={M} N={N} K={K} layout={layout} f16={f16}", flush=True)
    A, Bkn, sa, sb = make_problem(M + 5 * N + K, M, N, K, f16)
    st = np.float16 if f16 else np.float32
    dA, dB, dsa, dsb = dev(A), dev(b_of(Bkn, layout)), dev(sa.astype(st)), dev(sb.astype(st))
    bias = torch.linspace(-0.5, 0.5, N).cuda()
    biasmax = bias.abs().max().reshape(1)
    for rounding in (jf.ROUND_NEAREST, jf.ROUND_STOCHASTIC):
        q, s = jf.igemm_block_q(dA, dB, dsa, dsb, layout, rounding=rounding, seed=21, offset=8)
        assert q.cpu().numpy().any()
        for odt in (torch.float16, torch.bfloat16, torch.float32):
            got = jf.igemm_block_q_dequant(dA, dB, dsa, dsb, layout, out_dtype=odt, rounding=rounding, seed=21, offset=8)
            want = jf.dequantize(q, s, out_dtype=odt)
            assert got.dtype == odt and torch.equal(got.view(torch.int16 if odt != torch.float32 else torch.int32),
                                                    want.view(torch.int16 if odt != torch.float32 else torch.int32))
        wq, ws = oracle.igemm_block_q(A, Bkn, sa, sb, 1, stochastic=rounding == jf.ROUND_STOCHASTIC, seed=21, offset=8,
                                      scale_dtype="f16" if f16 else "f32")
        want32 = (wq.astype(np.float32).reshape(M // QB, QB, N // QB, QB) * ws.astype(np.float32)[:, None, :, None]).reshape(M, N)
        got32 = jf.igemm_block_q_dequant(dA, dB, dsa, dsb, layout, out_dtype=torch.float32, rounding=rounding, seed=21, offset=8)
        same(got32, want32, "dequantised result")
    # with a bias and its maximum (deterministic forward form), default output type = the scales' type
    qb, sbb = jf.igemm_block_q(dA, dB, dsa, dsb, layout, bias=bias, biasmax=biasmax)
    gotb = jf.igemm_block_q_dequant(dA, dB, dsa, dsb, layout, bias=bias, biasmax=biasmax)
    assert gotb.dtype == dsa.dtype and torch.equal(gotb, jf.dequantize(qb, sbb, out_dtype=dsa.dtype))
    with pytest.raises(RuntimeError):
        jf.igemm_block_q_dequant(dA, dB, dsa, dsb, layout, out_dtype=torch.float64)


@pytest.mark.gpu
def test_phase_recording_build_gives_the_same_bits_and_ordered_phases(jf):
    """The profiling build of the requantising GEMM (jf_prof_igemm_block_q of the measurement library) stores the same
    codes and scales as the product library's kernel, and every workgroup's phase stamps are in order with a plausible
    shader clock."""
    g = torch.Generator().manual_seed(5)
    M, N, K = 384, 416, 256                                     # 3 x 4 tiles, the last tile column a quarter full
    A = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8).cuda()
    B = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).cuda()
    sa = (torch.rand(K // 32, M // 32, generator=g) * 0.01 + 1e-3).cuda()
    sb = (torch.rand(K // 32, N // 32, generator=g) * 0.01 + 1e-3).cuda()
    for rounding, kw in ((jf.ROUND_NEAREST, {}), (jf.ROUND_STOCHASTIC, dict(seed=3, offset=8))):
        q0, s0 = jf.igemm_block_q(A, B, sa, sb, jf.B_NK, rounding=rounding, **kw)
        q, s, ph = jf.igemm_phases(A, B, sa, sb, jf.B_NK, rounding=rounding, **kw)
        assert torch.equal(q, q0) and torch.equal(s, s0)
        us = ph["us"]
        assert us.shape == (12, 6) and (us[:, 1:] >= us[:, :-1]).all() and us[:, 5].max() < 1e4
        assert ((ph["k_loop_MHz"] > 300) & (ph["k_loop_MHz"] < 3500)).all()
