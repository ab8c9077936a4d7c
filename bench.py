#!/usr/bin/env python3
"""Benchmark of the per-block INT8 linear path on one MI355X.

A step = one pass of the hot path over one batch of synthetic input at the GPT-2 XL shapes
(8192 tokens; QKV 1600->4800, proj 1600->1600, fc 1600->6400, fc2 6400->1600): for each of the four
linears the forward GEMM (INT8 requantised output), the dgrad GEMM (stochastic-rounding output) and the
wgrad GEMM (fp16 output) -- 12 fused per-block INT8 GEMMs, 1.51e12 integer ops.  Operands are
quantised once, outside the timed region, and stay resident in HBM.

Prints ONE JSON line: whole-step throughput as `value` (tera-ops/s), the roofline of the dominant
kernel (igemm_nt_kernel, measured live with events on the launch stream) and a CPU baseline (the CPU
checker under oracle/ timed on this host's cores on a bounded slice of the same workload).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "jetfire-int8training_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)

INT8_PEAK_TOPS = 5000.0      # MI355X dense INT8 MFMA peak, tera-ops/s
MEASURED_TRAFFIC_BYTES = 150.2e6   # fc forward GEMM: 97.3 MB fetched + 52.8 MB written per launch (counter run)
TOKENS = 8192
LAYERS = [("qkv", 1600, 4800), ("proj", 1600, 1600), ("fc", 1600, 6400), ("fc2", 6400, 1600)]


def make_inputs(jf, torch, seed=0):
    """BASELINE config 3: activations ~N(0,1) with 1% of channels x20, weights ~N(0,0.02), grads ~N(0,1e-3);
    all block-quantised with fp32 scales (gradients with stochastic rounding)."""
    g = torch.Generator().manual_seed(seed)
    ops = []
    for name, cin, cout in LAYERS:
        x = torch.randn(TOKENS, cin, generator=g)
        idx = torch.randperm(cin, generator=g)[: (cin + 99) // 100]
        x[:, idx] *= 20
        w = torch.randn(cout, cin, generator=g) * 0.02
        dy = torch.randn(TOKENS, cout, generator=g) * 1e-3
        qx, sx = jf.quantize(x.cuda(), scale_dtype=torch.float32)
        qw, sw = jf.quantize(w.cuda(), scale_dtype=torch.float32)
        qg, sg, qgT = jf.quantize(dy.cuda(), rounding=jf.ROUND_STOCHASTIC, scale_dtype=torch.float32,
                                  transpose=True, seed=seed, offset=0)
        ops.append(dict(name=name, cin=cin, cout=cout, qx=qx, sx=sx, sxT=sx.t().contiguous(), qw=qw, sw=sw,
                        swT=sw.t().contiguous(), qg=qg, sg=sg, sgT=sg.t().contiguous(), qgT=qgT))
    torch.cuda.synchronize()
    return ops


def step(jf, torch, ops, it):
    outs = []
    for o in ops:
        # forward  Y = X W^T           (M,N,K) = (T, cout, cin), B = W as [N,K]
        outs.append(jf.igemm_block_q(o["qx"], o["qw"], o["sxT"], o["swT"], jf.B_NK))
        # dgrad    dX = dY W           (T, cin, cout), B = W as [K,N], stochastic rounding
        outs.append(jf.igemm_block_q(o["qg"], o["qw"], o["sgT"], o["sw"], jf.B_KN, rounding=jf.ROUND_STOCHASTIC,
                                     seed=1234, offset=it * 7))
        # wgrad    dW = dY^T X         (cout, cin, T), A = dY^T, B = X as [K,N], fp16 out
        outs.append(jf.igemm_block_fp(o["qgT"], o["qx"], o["sg"], o["sx"], jf.B_KN, torch.float16))
    return outs


def step_ops():
    return sum(3 * 2 * TOKENS * cin * cout for _, cin, cout in LAYERS)


def dominant_kernel_roofline(jf, torch, ops, iters=20):
    """igemm_nt_kernel on the fc forward GEMM (8192 x 6400 x 1600, both operands K-contiguous, so the call is
    exactly one launch of that kernel): average launch duration from events on the launch stream."""
    o = ops[2]
    M, N, K = TOKENS, o["cout"], o["cin"]
    for _ in range(3):
        jf.igemm_block_q(o["qx"], o["qw"], o["sxT"], o["swT"], jf.B_NK)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        jf.igemm_block_q(o["qx"], o["qw"], o["sxT"], o["swT"], jf.B_NK)
    e1.record()
    torch.cuda.synchronize()
    avg_s = e0.elapsed_time(e1) * 1e-3 / iters
    achieved = 2.0 * M * N * K / avg_s / 1e12
    return {"bound": "mfma", "kernel": "igemm_nt_kernel<EPI_Q,f32> fc forward 8192x6400x1600",
            "achieved": round(achieved, 2), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
            "frac": round(achieved / INT8_PEAK_TOPS, 4), "avg_launch_us": round(avg_s * 1e6, 2),
            # HBM-side bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (profiles/igemm_fc_forward_pmc.md);
            # algorithmic minimum is 75.9 MB (A + W + C)
            "traffic": MEASURED_TRAFFIC_BYTES}


def fused_fc_gelu(jf, torch, ops):
    """The fc forward GEMM followed by the GELU kernel against the GEMM with the GELU in its epilogue (same bits)."""
    o = ops[2]
    sx, sw = o["sx"].t(), o["sw"].t()

    def separate():
        q, s = jf.igemm_block_q(o["qx"], o["qw"], sx, sw, jf.B_NK)
        return jf.gelu_fwd(q, s)

    out = {}
    for key, fn in (("gemm_then_gelu_us", separate), ("fused_us", lambda: jf.igemm_block_q_gelu(o["qx"], o["qw"], sx, sw))):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            fn()
        e1.record()
        torch.cuda.synchronize()
        out[key] = round(e0.elapsed_time(e1) * 1e3 / 20, 1)
    return out


def deep_k_weight_gradients(jf, torch):
    """Weight gradients of BASELINE config 2 (GPT-2 small, 12288 tokens) and the smallest one of the XL set: few output
    tiles over a deep K.  One accumulation chain per output (the reference's arithmetic) against the library's K split
    (ordered fp32 partial sums, `splitk=0`); both read the gradient [tokens, C_out] in place."""
    out = {}
    for name, T, cout, cin in (("gpt2small_qkv", 12288, 2304, 768), ("gpt2small_proj", 12288, 768, 768),
                               ("gpt2small_fc", 12288, 3072, 768), ("gpt2small_fc2", 12288, 768, 3072),
                               ("xl_proj", TOKENS, 1600, 1600)):
        g = torch.randint(-127, 128, (T, cout), dtype=torch.int8, device="cuda")
        x = torch.randint(-127, 128, (T, cin), dtype=torch.int8, device="cuda")
        sg = torch.rand(T // 32, cout // 32, device="cuda") + 0.5
        sx = torch.rand(T // 32, cin // 32, device="cuda") + 0.5
        r = {"parts": jf.splitk_plan(cout, cin, T, 0)[0]}
        for key, sk in (("one_chain", 1), ("split_k", 0)):
            for _ in range(3):
                jf.igemm_block_fp(g, x, sg, sx, jf.B_KN, torch.float16, a_layout=jf.A_KM, splitk=sk)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(20):
                jf.igemm_block_fp(g, x, sg, sx, jf.B_KN, torch.float16, a_layout=jf.A_KM, splitk=sk)
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / 20
            r[key] = {"us": round(us, 1), "TOP/s": round(2.0 * T * cout * cin / us / 1e6, 1)}
        out[f"{name}_{cout}x{cin}x{T}"] = r
    return out


def recipe_block(torch):
    """One GPT-2 XL transformer block (1600 wide, 25 heads) forward + backward on 8 x 1024 tokens: the INT8 data-flow
    recipe (Jetfire/recipe.py: every linear layer, LayerNorm, GELU and residual add on INT8 block tensors, attention
    itself in fp16 through torch) next to the same block in plain torch bf16."""
    import torch.nn.functional as F
    sys.path.insert(0, os.path.join(PKG, "Jetfire"))
    from recipe import QStack
    torch.manual_seed(0)
    B, T, C, H = 8, 1024, 1600, 25
    model = QStack(1, C, H).cuda()
    blk = model.blocks[0]
    x = torch.randn(B, T, C, device="cuda", requires_grad=True)
    w = torch.randn(B, T, C, device="cuda")

    def ref_block(xr, dt):
        h = F.layer_norm(xr, (C,), blk.ln_1.to(dt), None, 1e-5)
        qkv = h @ blk.w_qkv.to(dt).t()
        q, k, v = (t.view(B, T, H, C // H).transpose(1, 2) for t in qkv.split(C, dim=2))
        y = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).contiguous().view(B, T, C)
        xr = xr + y @ blk.w_attn_proj.to(dt).t()
        h = F.layer_norm(xr, (C,), blk.ln_2.to(dt), None, 1e-5)
        return xr + F.gelu(h @ blk.w_fc.to(dt).t()) @ blk.w_mlp_proj.to(dt).t()

    def t(fn, n=10):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return round(e0.elapsed_time(e1) / n, 3)

    xr, wr = x.detach().to(torch.bfloat16).requires_grad_(True), w.to(torch.bfloat16)
    return {"tokens": B * T, "int8_recipe_ms": t(lambda: model(x).backward(w)),
            "torch_bf16_ms": t(lambda: ref_block(xr, torch.bfloat16).backward(wr))}


def nonlinear_extras(jf, torch):
    """Achieved GB/s (algorithmic bytes / event time) of the memory-bound kernels at the GPT-2 XL sizes of BASELINE
    config 4 (LayerNorm on 8192x1600, GELU on 8192x6400), fp32 scales."""
    def t(fn, n=20, replays=5):
        """Seconds per call.  Several of these kernels run for 5-15 us, less than one call of the Python wrapper
        costs on the host, so the launches are recorded into a HIP graph once and the replays are timed (events on
        the replay stream); eager back-to-back launches are the fallback."""
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(n):
                    fn()
            graph.replay()
            torch.cuda.synchronize()
            e0.record()
            for _ in range(replays):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e-3 / (n * replays)
        except Exception:
            torch.cuda.synchronize()
            e0.record()
            for _ in range(n):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e-3 / n
    g = torch.Generator().manual_seed(0)
    S = torch.float32
    out = {}
    def put(name, secs, nbytes):
        out[name] = {"GB/s": round(nbytes / secs / 1e9, 1), "us": round(secs * 1e6, 1), "frac_of_8TB/s": round(nbytes / secs / 8e12, 3)}
    R, C = TOKENS, 1600
    x = torch.randn(R, C, generator=g).cuda()
    dy = (torch.randn(R, C, generator=g) * 1e-3).cuda()
    gamma = (1 + 0.1 * torch.randn(C, generator=g)).cuda()
    beta = (0.1 * torch.randn(C, generator=g)).cuda()
    qx, sx = jf.quantize(x, scale_dtype=S)
    qg, sg = jf.quantize(dy, jf.ROUND_STOCHASTIC, S, seed=0, offset=0)
    mean, rstd = jf.rowstats(qx, sx)
    n = R * C
    put("quantize_f32_8192x1600", t(lambda: jf.quantize(x, scale_dtype=S)), 5 * n)
    put("quantize_transpose_sr_8192x1600", t(lambda: jf.quantize(x, jf.ROUND_STOCHASTIC, S, transpose=True, seed=1, offset=0)), 6 * n)
    put("transpose_8192x1600", t(lambda: jf.transpose_s8(qx)), 2 * n)
    put("layernorm_fwd_8192x1600", t(lambda: jf.layernorm_fwd(qx, sx, gamma, beta, mean, rstd)), 2 * n)
    put("layernorm_bwd_sr_8192x1600", t(lambda: jf.layernorm_bwd(qx, sx, qg, sg, gamma, mean, rstd, jf.ROUND_STOCHASTIC, seed=1, offset=0)), 3 * n)
    R, C = TOKENS, 6400
    x = torch.randn(R, C, generator=g).cuda()
    dy = (torch.randn(R, C, generator=g) * 1e-3).cuda()
    qx, sx = jf.quantize(x, scale_dtype=S)
    qg, sg = jf.quantize(dy, jf.ROUND_STOCHASTIC, S, seed=0, offset=0)
    n = R * C
    put("gelu_fwd_tanh_8192x6400", t(lambda: jf.gelu_fwd(qx, sx, jf.GELU_TANH, 0.0)), 2 * n)
    put("gelu_fwd_erf_8192x6400", t(lambda: jf.gelu_fwd(qx, sx, jf.GELU_ERF, 5e-5)), 2 * n)
    put("gelu_bwd_tanh_sr_8192x6400", t(lambda: jf.gelu_bwd(qx, sx, qg, sg, jf.GELU_TANH, jf.ROUND_STOCHASTIC, seed=1, offset=0)), 3 * n)
    put("gelu_bwd_erf_sr_8192x6400", t(lambda: jf.gelu_bwd(qx, sx, qg, sg, jf.GELU_ERF, jf.ROUND_STOCHASTIC, seed=1, offset=0)), 3 * n)
    return out


def calibration(jf, torch):
    """Register-only loops: what the matrix pipe and the vector ALU deliver alone and together on this part."""
    simds = torch.cuda.get_device_properties(0).multi_processor_count * 4
    out = {}
    t, n = jf.calibrate(1, 0)
    out["mfma_only_TOPs"] = round(n * 65536 / t / 1e12, 1)
    out["mfma_only_ns_per_mfma_per_simd"] = round(t * 1e9 * simds / n, 2)
    t, n = jf.calibrate(0, 32)
    out["valu_32fmac_ns_per_simd"] = round(t * 1e9 * simds / n, 2)
    t, n = jf.calibrate(1, 32)
    out["mfma_plus_32fmac_ns_per_simd"] = round(t * 1e9 * simds / n, 2)
    out["mfma_plus_32fmac_TOPs"] = round(n * 65536 / t / 1e12, 1)
    a = torch.randn(TOKENS, 1600, device="cuda", dtype=torch.bfloat16)
    b = torch.randn(6400, 1600, device="cuda", dtype=torch.bfloat16)
    for _ in range(5):
        a @ b.t()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        a @ b.t()
    e1.record()
    torch.cuda.synchronize()
    out["torch_bf16_fc_forward_TFLOPs"] = round(2.0 * TOKENS * 6400 * 1600 * 20 / (e0.elapsed_time(e1) * 1e-3) / 1e12, 1)
    out["note"] = ("per SIMD, 4 waves resident; the scale-accumulate needs 32 VALU instructions per MFMA, and the two "
                   "pipes add up rather than overlap: the last line is the ceiling of any exact per-block kernel")
    return out


def pmc_probe(jf, torch, ops):
    """For counter runs (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE): one device copy of known size (256 MiB read,
    256 MiB written: the calibration kernel) followed by three launches of the dominant GEMM, and nothing else."""
    buf = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(buf)
    torch.cuda.synchronize()
    dst.copy_(buf)
    o = ops[2]
    for _ in range(3):
        jf.igemm_block_q(o["qx"], o["qw"], o["sxT"], o["swT"], jf.B_NK)
    torch.cuda.synchronize()


def cpu_baseline(ops, rows=512):
    """The CPU checker (scalar C restatement of the reference arithmetic, OpenMP over rows) on the first
    `rows` token rows of the fc layer: forward + dgrad + the matching slice of wgrad work."""
    import numpy as np
    from oracle import oracle as O
    threads = min(os.cpu_count() or 1, 16)
    O.set_threads(threads)
    o = ops[2]
    f = lambda t: np.ascontiguousarray(t.cpu().numpy())
    qx, qw, qg = f(o["qx"][:rows]), f(o["qw"]), f(o["qg"][:rows])
    sxT, swT, sgT, sw = f(o["sxT"][:, : rows // 32]), f(o["swT"]), f(o["sgT"][:, : rows // 32]), f(o["sw"])
    qgT, sg, sx = f(o["qgT"][:, :rows]), f(o["sg"][: rows // 32]), f(o["sx"][: rows // 32])
    t0 = time.perf_counter()
    O.igemm_block_q(qx, qw, sxT, swT, 0)
    O.igemm_block_q(qg, qw, sgT, sw, 1, stochastic=True, seed=1234, offset=0)
    O.igemm_block_fp(qgT, qx, sg, sx, 1, "f16")
    dt = time.perf_counter() - t0
    nops = 3 * 2.0 * rows * o["cin"] * o["cout"]
    return {"value": round(nops / dt / 1e12, 5), "unit": "TOP/s", "cores": threads, "kind": "port",
            "sample": f"fc layer (1600->6400), first {rows} of 8192 token rows: forward + dgrad(SR) + wgrad slice, "
                      f"{nops:.3g} ops in {dt:.1f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--cpu-rows", type=int, default=8192)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--pmc-probe", action="store_true", help="copy kernel + 3 GEMM launches only (for rocprofv3 --pmc)")
    ap.add_argument("--roofline-only", action="store_true", help="only the dominant-kernel measurement (for rocprofv3 --stats)")
    ap.add_argument("--extras-only", action="store_true", help="only the block-kernel section (for rocprofv3 --pmc)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (--gpus 1); nothing here uses a second GPU")

    import torch
    import jetfire_hip as jf
    jf.lib()
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    torch.cuda.set_device(0)
    ops = make_inputs(jf, torch)
    if a.pmc_probe:
        pmc_probe(jf, torch, ops)
        return
    if a.roofline_only:
        print(json.dumps({"roofline": dominant_kernel_roofline(jf, torch, ops)}))
        return
    if a.extras_only:
        print(json.dumps({"memory_bound_kernels": nonlinear_extras(jf, torch)}))
        return

    for i in range(a.warmup):
        step(jf, torch, ops, i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(a.steps):
        step(jf, torch, ops, a.warmup + i)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = wall * 1e3 / a.steps
    tops = step_ops() / (wall / a.steps) / 1e12

    roof = dominant_kernel_roofline(jf, torch, ops)
    out = {
        "metric": "per-block INT8 GEMM TOPS (% of INT8 MFMA peak) fwd+bwd at GPT-2 XL shapes",
        "value": round(tops, 2), "unit": "TOPS", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 (int32 block accumulate, fp32 scale-accumulate)", "data": "synthetic",
        "config": {"workload": "GPT-2 XL linear set, 8192 tokens: {qkv 1600->4800, proj 1600->1600, fc 1600->6400, "
                               "fc2 6400->1600} x {forward (requantised), dgrad (stochastic), wgrad (fp16)}, "
                               "32x32 per-block INT8, fp32 scales, 1% outlier channels x20",
                   "ops_per_step": step_ops(), "pct_of_int8_peak": round(100 * tops / INT8_PEAK_TOPS, 2),
                   "event_ms_per_step": round(e0.elapsed_time(e1) / a.steps, 4)},
        "roofline": roof,
    }
    if not a.no_extras:
        out["calibration"] = calibration(jf, torch)
        out["memory_bound_kernels"] = nonlinear_extras(jf, torch)
        out["deep_k_weight_gradients"] = deep_k_weight_gradients(jf, torch)
        out["fc_forward_with_gelu"] = fused_fc_gelu(jf, torch, ops)
        out["xl_block_forward_backward"] = recipe_block(torch)
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline(ops, a.cpu_rows)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
