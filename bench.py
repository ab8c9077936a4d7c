#!/usr/bin/env python3
"""Benchmark of the per-block INT8 linear path on one MI355X.

A step = one pass of the hot path over one batch of synthetic input at the GPT-2 XL shapes
(8192 tokens; QKV 1600->4800, proj 1600->1600, fc 1600->6400, fc2 6400->1600): for each of the four
linears the forward GEMM (INT8 requantised output), the dgrad GEMM (stochastic-rounding output) and the
wgrad GEMM (fp16 output) -- 12 fused per-block INT8 GEMMs, 1.51e12 integer ops.  Operands are
quantised once, outside the timed region, and stay resident in HBM.

Prints ONE JSON line: whole-step throughput as `value` (tera-ops/s), the roofline of the dominant
kernel (igemm_nt_kernel, measured live with events on the launch stream) and a CPU baseline (a PyTorch
emulation of the same arithmetic, and the C restatement under oracle/, timed on this host's cores on a
bounded slice of the same workload).
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
# HBM-side bytes per launch of the fc forward GEMM, from the rocprofv3 --pmc runs summarised in
# profiles/igemm_fc_forward_pmc.md (FETCH_SIZE and WRITE_SIZE, each scaled by a copy of known size): a property of the
# kernel, carried over from that profile, not re-measured by this run (counters need the profiler attached)
PROFILED_TRAFFIC_BYTES = 160.3e6
PROFILED_TRAFFIC_SOURCE = "profiles/igemm_fc_forward_pmc.md (101.0 MB fetched + 59.3 MB written; algorithmic 75.9 MB)"
TOKENS = 8192
LAYERS = [("qkv", 1600, 4800), ("proj", 1600, 1600), ("fc", 1600, 6400), ("fc2", 6400, 1600)]


def make_inputs(jf, torch, seed=0):
    """benchmark configuration 3: activations ~N(0,1) with 1% of channels x20, weights ~N(0,0.02), grads ~N(0,1e-3);
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
    offset = it * (sum(TOKENS * o["cin"] for o in ops) // 8)      # every dgrad launch of the run draws its own counters
    for o in ops:
        # forward  Y = X W^T           (M,N,K) = (T, cout, cin), B = W as [N,K]
        outs.append(jf.igemm_block_q(o["qx"], o["qw"], o["sxT"], o["swT"], jf.B_NK))
        # dgrad    dX = dY W           (T, cin, cout), B = W as [K,N], stochastic rounding
        outs.append(jf.igemm_block_q(o["qg"], o["qw"], o["sgT"], o["sw"], jf.B_KN, rounding=jf.ROUND_STOCHASTIC,
                                     seed=1234, offset=offset))
        offset += TOKENS * o["cin"] // 8
        # wgrad    dW = dY^T X         (cout, cin, T), A = dY^T, B = X as [K,N], fp16 out
        outs.append(jf.igemm_block_fp(o["qgT"], o["qx"], o["sg"], o["sx"], jf.B_KN, torch.float16))
    return outs


def step_ops():
    return sum(3 * 2 * TOKENS * cin * cout for _, cin, cout in LAYERS)


def dominant_kernel_roofline(jf, torch, ops, iters=200):
    """igemm_nt_kernel on the fc forward GEMM (8192 x 6400 x 1600, both operands K-contiguous, so the call is
    exactly one launch of that kernel): average launch duration from events on the launch stream."""
    o = ops[2]
    M, N, K = TOKENS, o["cout"], o["cin"]
    # The clocks under this load settle only after a few tenths of a second of sustained work (shader clock 1.87 GHz in a
    # process that starts timing at once, 2.0-2.08 GHz after 0.3 s; a compute-only warm-up raises the shader clock but
    # leaves the first launches slow all the same): hold the GPU busy first with the same GEMM through another instantiation
    # of the kernel (the one with the GELU epilogue), so that a kernel trace of this command lists the timed launches alone
    for _ in range(1500):
        jf.igemm_block_q_gelu(o["qx"], o["qw"], o["sxT"], o["swT"])
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
    # the same launch once more, right behind the timed ones (the clock has settled), with the kernel's profiling build:
    # when each workgroup's phases began and ended and the shader clock its main loop ran at
    tiles = ((M + 127) // 128) * ((N + 127) // 128)
    _, _, ph = jf.igemm_phases(o["qx"], o["qw"], o["sxT"], o["swT"], jf.B_NK)
    us, mhz = ph["us"], float(ph["k_loop_MHz"].mean())
    span_us = float(us[:, 5].max())
    products = (M // 32) * (N // 32) * (K // 32)              # 32x32x32 block products = MFMA instructions
    simds = 4 * torch.cuda.get_device_properties(0).multi_processor_count
    d = us[:, 1:] - us[:, :-1]
    phases = {"workgroups": tiles, "span_us": round(span_us, 1), "main_loop_shader_MHz": round(mhz),
              "simd_cycles_per_block_product": round(avg_s * 1e6 * mhz * simds / products, 1),
              "mean_us": {k: round(float(d[:, i].mean()), 2) for i, k in
                          enumerate(("prologue", "main_loop", "sync", "requantise", "store"))},
              "note": "simd_cycles_per_block_product = average launch time (of the normal build, above) x this clock x "
                      "SIMDs / MFMA count: everything the kernel does, per MFMA; span_us is the recorded launch alone, first "
                      "workgroup start to last workgroup end; the register-only stream of one MFMA + 32 VALU instructions takes the cycles the calibration "
                      "table gives for gemm_k_block_stream"}
    return {"bound": "mfma", "kernel": "igemm_nt_kernel<EPI_Q,f32> fc forward 8192x6400x1600",
            "achieved": round(achieved, 2), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
            "frac": round(achieved / INT8_PEAK_TOPS, 4), "avg_launch_us": round(avg_s * 1e6, 2),
            "launches": iters, "traffic": PROFILED_TRAFFIC_BYTES, "traffic_carried_from_profile": True,
            "traffic_source": PROFILED_TRAFFIC_SOURCE, "phases": phases}


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


def fused_fc2_dgrad_gelu_bwd(jf, torch, ops):
    """The fc2 activation-gradient GEMM followed by the GELU backward kernel against the GEMM with the GELU backward in
    its epilogue (same bits); the layer's quantised input stands in for the GELU's saved input (same shape)."""
    o = ops[3]                                                     # fc2: 6400 -> 1600, so dX is [8192, 6400]
    sg, sw = o["sg"].t(), o["sw"]

    def separate():
        q, s = jf.igemm_block_q(o["qg"], o["qw"], sg, sw, jf.B_KN, rounding=jf.ROUND_STOCHASTIC, seed=1, offset=0)
        return jf.gelu_bwd(o["qx"], o["sx"], q, s, jf.GELU_ERF, jf.ROUND_STOCHASTIC, seed=2, offset=0)

    def fused():
        return jf.igemm_block_q_gelu_bwd(o["qg"], o["qw"], sg, sw, o["qx"], o["sx"], jf.GELU_ERF, jf.ROUND_STOCHASTIC,
                                         seed=1, offset=0, gelu_seed=2, gelu_offset=0)
    return {"gemm_then_gelu_bwd_us": round(timed_us(torch, separate, 30), 1), "fused_us": round(timed_us(torch, fused, 30), 1)}


def deep_k_weight_gradients(jf, torch):
    """Weight gradients of benchmark configuration 2 (GPT-2 small, 12288 tokens) and the smallest one of the XL set: few output
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


def recipe_block(torch, only=None, shape=(8, 1024, 1600, 25)):
    """Transformer blocks forward + backward, by default GPT-2 XL's (1600 wide, 25 heads) on 8 x 1024 tokens; shape =
    (12, 1024, 768, 12) is GPT-2 small's on 12288 tokens, where kernels are short and host overhead shows: the INT8 data-flow
    recipe (Jetfire/recipe.py: every linear layer, LayerNorm, GELU and residual add on INT8 block tensors, attention
    itself in fp16 through torch) next to the same blocks in plain torch bf16.  Measured for a stack of one block (which
    includes the stack's own begin / end: quantising the input, its row statistics, quantising the output gradient) and
    of three; the difference, halved, is what a block costs inside a stack.  Parameter gradients are reset to None before
    every step, as an optimizer's zero_grad() does.  The INT8 stack takes a float32 input (an embedding's output) and
    carries a bfloat16 residual between blocks, as the reference does (INT8_GPT2/qmodel.py:228); the sum inside a block
    stays float32.  Both sides pay for their weights in every step: the INT8 stack quantises them again (its cache of weight
    codes is cleared, as after an optimizer update), the bf16 blocks cast them."""
    import torch.nn.functional as F
    sys.path.insert(0, os.path.join(PKG, "Jetfire"))
    from recipe import QStack, weight_codes
    torch.manual_seed(0)
    B, T, C, H = shape
    x = torch.randn(B, T, C, device="cuda", requires_grad=True)
    w = torch.randn(B, T, C, device="cuda")
    xr, wr = x.detach().to(torch.bfloat16).requires_grad_(True), w.to(torch.bfloat16)

    def t(fn, params, n=10):
        def step():
            for p in params:
                p.grad = None
            fn()
        for _ in range(3):
            step()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            step()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    out = {}
    for layers in ((3,) if only else (1, 3)):
        model = QStack(layers, C, H, stream_dtype=torch.bfloat16).cuda()    # fp32 in, bfloat16 between blocks and out

        def ref_stack(h0, dt):
            for blk in model.blocks:
                h = F.layer_norm(h0, (C,), blk.ln_1.to(dt), None, 1e-5)
                qkv = h @ blk.w_qkv.to(dt).t()
                q, k, v = (u.view(B, T, H, C // H).transpose(1, 2) for u in qkv.split(C, dim=2))
                y = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).contiguous().view(B, T, C)
                h0 = h0 + y @ blk.w_attn_proj.to(dt).t()
                h = F.layer_norm(h0, (C,), blk.ln_2.to(dt), None, 1e-5)
                h0 = h0 + F.gelu(h @ blk.w_fc.to(dt).t()) @ blk.w_mlp_proj.to(dt).t()
            return h0
        params = list(model.parameters())

        def int8_step():
            # a training step follows an optimizer update: the cached weight codes are stale and every weight is quantised
            # again (the bf16 blocks cast their weights in every step as well)
            weight_codes.clear()
            model(x).backward(wr)

        def peak_mb(fn):
            # memory held at the end of the forward pass above what is held before it (saved activations + output)
            for q in params + [x, xr]:
                q.grad = None
            torch.cuda.synchronize()
            base = torch.cuda.memory_allocated()
            y = fn()
            torch.cuda.synchronize()
            held = torch.cuda.memory_allocated() - base
            y.backward(w if y.dtype == w.dtype else wr)
            del y
            return round(held / 2 ** 20, 1)
        if layers == 3 and not only:
            out["mem"] = (peak_mb(lambda: model(x)), peak_mb(lambda: ref_stack(xr, torch.bfloat16)))
        if only:                                                   # one of the two, 3 + 10 steps: a kernel trace of it
            return round(t(int8_step, params + [x]) if only == "int8"
                         else t(lambda: ref_stack(xr, torch.bfloat16).backward(wr), params + [xr]), 3)
        if layers == 3:                                            # weight codes reused between steps (micro-batches of one update)
            out["cached"] = t(lambda: model(x).backward(wr), params + [x])
        out[layers] = (t(int8_step, params + [x]),
                       t(lambda: ref_stack(xr, torch.bfloat16).backward(wr), params + [xr]))
        del model
    return {"tokens": B * T, "int8_recipe_ms": round(out[1][0], 3), "torch_bf16_ms": round(out[1][1], 3),
            "stack_of_3_blocks": {"int8_recipe_ms": round(out[3][0], 3), "torch_bf16_ms": round(out[3][1], 3),
                                  "int8_recipe_weight_codes_reused_ms": round(out["cached"], 3),
                                  "held_after_forward_MiB": {"int8_recipe": out["mem"][0], "torch_bf16": out["mem"][1]}},
            "per_block_inside_a_stack": {"int8_recipe_ms": round((out[3][0] - out[1][0]) / 2, 3),
                                         "torch_bf16_ms": round((out[3][1] - out[1][1]) / 2, 3)}}


def nonlinear_extras(jf, torch):
    """Achieved GB/s (algorithmic bytes / event time) of the memory-bound kernels at the GPT-2 XL sizes of benchmark
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
    COLD_BYTES = 320 << 20         # more than the 256 MiB Infinity Cache between two uses of the same bytes

    def put(name, secs, nbytes, cold=None):
        """cold = (fn(inputs), inputs): the same call timed again while rotating over as many clones of its input tensors
        as it takes for COLD_BYTES of other operands to pass between two uses of a clone (outputs are fresh buffers in
        either measurement), so that every byte comes from and goes to HBM: GB/s_cold / frac_cold.  The first figures
        replay one set of inputs (<= 157 MB, cache-warm reads): an upper bound."""
        out[name] = {"GB/s": round(nbytes / secs / 1e9, 1), "us": round(secs * 1e6, 1), "frac_of_8TB/s": round(nbytes / secs / 8e12, 3)}
        if cold is not None:
            fn, inputs = cold
            in_bytes = sum(t.numel() * t.element_size() for t in inputs)
            sets = [inputs] + [tuple(t.clone() for t in inputs) for _ in range(max(2, -(-COLD_BYTES // max(in_bytes, 1))))]
            state = {"i": 0}

            def rotating():
                fn(*sets[state["i"] % len(sets)])
                state["i"] += 1
            n = 2 * len(sets)
            state["i"] = 0
            secs_cold = t(rotating, n=n, replays=3)
            out[name].update({"us_cold": round(secs_cold * 1e6, 1), "GB/s_cold": round(nbytes / secs_cold / 1e9, 1),
                              "frac_cold": round(nbytes / secs_cold / 8e12, 3), "input_sets": len(sets)})
    R, C = TOKENS, 1600
    x = torch.randn(R, C, generator=g).cuda()
    dy = (torch.randn(R, C, generator=g) * 1e-3).cuda()
    gamma = (1 + 0.1 * torch.randn(C, generator=g)).cuda()
    beta = (0.1 * torch.randn(C, generator=g)).cuda()
    qx, sx = jf.quantize(x, scale_dtype=S)
    qg, sg = jf.quantize(dy, jf.ROUND_STOCHASTIC, S, seed=0, offset=0)
    mean, rstd = jf.rowstats(qx, sx)
    n = R * C
    f = lambda x_: jf.quantize(x_, scale_dtype=S)
    put("quantize_f32_8192x1600", t(lambda: f(x)), 5 * n, (f, (x,)))
    f = lambda x_: jf.quantize(x_, jf.ROUND_STOCHASTIC, S, transpose=True, seed=1, offset=0)
    put("quantize_transpose_sr_8192x1600", t(lambda: f(x)), 6 * n, (f, (x,)))
    f = lambda q_: jf.transpose_s8(q_)
    put("transpose_8192x1600", t(lambda: f(qx)), 2 * n, (f, (qx,)))
    f = lambda q_, s_: jf.layernorm_fwd(q_, s_, gamma, beta, mean, rstd)
    put("layernorm_fwd_8192x1600", t(lambda: f(qx, sx)), 2 * n, (f, (qx, sx)))
    f = lambda q_, s_, g_, sg_: jf.layernorm_bwd(q_, s_, g_, sg_, gamma, mean, rstd, jf.ROUND_STOCHASTIC, seed=1, offset=0)
    put("layernorm_bwd_sr_8192x1600", t(lambda: f(qx, sx, qg, sg)), 3 * n, (f, (qx, sx, qg, sg)))
    # residual add: fp32 in + codes in, fp32 out + codes out (the reference's default truncation; the backward's stochastic
    # form; the forward's form with the row partial sums and their finishing launch)
    f = lambda x_, q_, s_: jf.add(x_, q_, s_, jf.ROUND_TRUNC)
    put("add_8192x1600", t(lambda: f(x, qx, sx)), 10 * n, (f, (x, qx, sx)))
    f = lambda x_, q_, s_: jf.add(x_, q_, s_, jf.ROUND_STOCHASTIC_TRUNC, seed=1, offset=0)
    put("add_sr_8192x1600", t(lambda: f(x, qx, sx)), 10 * n, (f, (x, qx, sx)))
    f = lambda x_, q_, s_: jf.rowstats_finish(*jf.add(x_, q_, s_, jf.ROUND_TRUNC, with_stats=True)[3:], C)
    put("add_meanvar_8192x1600", t(lambda: f(x, qx, sx)), 10 * n, (f, (x, qx, sx)))
    # LayerNorm backward with the residual add behind it in one kernel (what the recipe's backward runs), fp32 / bfloat16
    # gradient in and out: codes of x and dy in; the fp gradient in; the sum and its codes out
    xb = x.to(torch.bfloat16)
    f = lambda q_, s_, g_, sg_, x_: jf.layernorm_bwd_add(q_, s_, g_, sg_, gamma, mean, rstd, x_, jf.ROUND_STOCHASTIC,
                                                         jf.ROUND_STOCHASTIC_TRUNC, seed=1, offset=0, add_seed=2, add_offset=0)
    put("layernorm_bwd_add_sr_8192x1600", t(lambda: f(qx, sx, qg, sg, x)), 11 * n, (f, (qx, sx, qg, sg, x)))
    f = lambda q_, s_, g_, sg_, x_: jf.layernorm_bwd_add(q_, s_, g_, sg_, gamma, mean, rstd, x_, jf.ROUND_STOCHASTIC,
                                                         jf.ROUND_STOCHASTIC_TRUNC, out_dtype=torch.bfloat16, seed=1, offset=0,
                                                         add_seed=2, add_offset=0)
    put("layernorm_bwd_add_sr_bf16_8192x1600", t(lambda: f(qx, sx, qg, sg, xb)), 7 * n, (f, (qx, sx, qg, sg, xb)))
    f = lambda g_, sg_: jf.block_colsum(g_, sg_)
    put("bias_gradient_colsum_8192x1600", t(lambda: f(qg, sg)), n, (f, (qg, sg)))
    # what a plain device copy of the same bytes reaches under the same two measurements (1 + 1 bytes per element, the
    # traffic of LayerNorm / GELU forward): the ceiling of this method at this size, beside the 8 TB/s the fractions use
    f = lambda q_: torch.empty_like(q_).copy_(q_)
    put("reference_copy_s8_8192x1600", t(lambda: f(qx)), 2 * n, (f, (qx,)))
    R, C = TOKENS, 6400
    x = torch.randn(R, C, generator=g).cuda()
    dy = (torch.randn(R, C, generator=g) * 1e-3).cuda()
    qx, sx = jf.quantize(x, scale_dtype=S)
    qg, sg = jf.quantize(dy, jf.ROUND_STOCHASTIC, S, seed=0, offset=0)
    n = R * C
    del x, dy
    f = lambda q_: torch.empty_like(q_).copy_(q_)
    put("reference_copy_s8_8192x6400", t(lambda: f(qx)), 2 * n, (f, (qx,)))
    f = lambda q_, s_: jf.gelu_fwd(q_, s_, jf.GELU_TANH, 0.0)
    put("gelu_fwd_tanh_8192x6400", t(lambda: f(qx, sx)), 2 * n, (f, (qx, sx)))
    f = lambda q_, s_: jf.gelu_fwd(q_, s_, jf.GELU_ERF, 5e-5)
    put("gelu_fwd_erf_8192x6400", t(lambda: f(qx, sx)), 2 * n, (f, (qx, sx)))
    f = lambda q_, s_, g_, sg_: jf.gelu_bwd(q_, s_, g_, sg_, jf.GELU_TANH, jf.ROUND_STOCHASTIC, seed=1, offset=0)
    put("gelu_bwd_tanh_sr_8192x6400", t(lambda: f(qx, sx, qg, sg)), 3 * n, (f, (qx, sx, qg, sg)))
    f = lambda q_, s_, g_, sg_: jf.gelu_bwd(q_, s_, g_, sg_, jf.GELU_ERF, jf.ROUND_STOCHASTIC, seed=1, offset=0)
    put("gelu_bwd_erf_sr_8192x6400", t(lambda: f(qx, sx, qg, sg)), 3 * n, (f, (qx, sx, qg, sg)))
    out["note"] = ("GB/s = algorithmic bytes / time.  The first figures replay one set of input tensors (reads served by the "
                   "256 MiB Infinity Cache where they fit): an upper bound.  *_cold rotate over clones of the inputs so that every "
                   "byte comes from HBM: the figure the 70 %-of-HBM target is judged on.")
    return out


def host_call_overhead(jf, torch):
    """Host microseconds per operator call on operands so small that the GPU never is the bottleneck (one 32 x 32 block):
    the Python ctypes binding of the C ABI (what the Nonlinear package called before) against the C++ extension (what it
    calls now), and the package-level functions on top of the extension."""
    sys.path.insert(0, os.path.join(PKG, "Jetfire"))
    import BlockQuantizeCUDA as BQC
    from Nonlinear import int8_gelu_forward, int8_quantize
    J = BQC.jetfire
    x = torch.randn(32, 32, device="cuda")
    q, s = jf.quantize(x)

    def per_call(fn, n=2000):
        for _ in range(50):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        dt = time.perf_counter() - t0
        torch.cuda.synchronize()
        return round(dt / n * 1e6, 2)
    return {"gelu_fwd": {"ctypes_binding_us": per_call(lambda: jf.gelu_fwd(q, s)), "cpp_extension_us": per_call(lambda: J.gelu_fwd(q, s)),
                         "Nonlinear.int8_gelu_forward_us": per_call(lambda: int8_gelu_forward(q, s, 32))},
            "quantize": {"ctypes_binding_us": per_call(lambda: jf.quantize(x)), "cpp_extension_us": per_call(lambda: J.quantize(x)),
                         "Nonlinear.int8_quantize_us": per_call(lambda: int8_quantize(x, 32))},
            "quantize_stochastic": {"ctypes_binding_us": per_call(lambda: jf.quantize(x, jf.ROUND_STOCHASTIC)),
                                    "cpp_extension_us": per_call(lambda: J.quantize(x, J.ROUND_STOCHASTIC))},
            "note": "wall time of back-to-back calls on one 32x32 block (launch-bound on the host side), 2000 calls"}


def calibration(jf, torch):
    """Register-only loops: what the matrix pipe and the vector ALU deliver alone, together in one wave, together from
    separate waves of one SIMD, and on the GEMM's real K-block instruction stream, at 1 / 2 / 4 waves per SIMD, in
    nanoseconds and in shader cycles (with the clock the kernel ran at) per work item and SIMD."""
    out = {"unit": "per 32x32x32 work item and SIMD", "rows": []}

    def row(name, *a, **kw):
        r = jf.calibrate(*a, **kw)
        ns = r["seconds"] * 1e9 * r["simds"] / r["items"]
        out["rows"].append({"case": name, "waves_per_simd": r["waves_per_simd"], "ns": round(ns, 2),
                            "cycles": round(ns * r["shader_MHz"] * 1e-3, 1), "shader_MHz": round(r["shader_MHz"])})
        return ns

    for wpc in (1, 2, 4):                                         # 256-thread workgroups: one wave per SIMD each
        row("mfma_only", 1, 0, workgroups_per_cu=wpc)
        row("valu_32fmac_only", 0, 32, workgroups_per_cu=wpc)
        both = row("mfma_and_32fmac_same_wave", 1, 32, workgroups_per_cu=wpc)
        stream = row("gemm_k_block_stream", 1, 32, workgroups_per_cu=wpc, mode=jf.CAL_STREAM)
    for wpc in (1, 2):                                            # 512-thread workgroups: waves w and w+4 share a SIMD
        row("mfma_and_32fmac_separate_waves", 1, 32, workgroups_per_cu=wpc, threads=512, mode=jf.CAL_SPLIT)
    # the same stream on operands that change with every MFMA and use all 8 bits, held for ~150 ms: the shader clock
    # depends on how much the datapaths toggle, and the first stream above runs on near-constant operands
    sustained = row("gemm_k_block_stream_changing_operands_sustained", 1, 32, iters=20000, workgroups_per_cu=2, threads=512,
                    mode=jf.CAL_STREAM_DATA, launches=10)
    out["ceiling_TOPs_independent"] = round(65536 / both * 1e9 * 1024 / 1e12, 1)
    out["ceiling_TOPs_k_block_stream"] = round(65536 / stream * 1e9 * 1024 / 1e12, 1)
    out["ceiling_TOPs_k_block_stream_changing_operands"] = round(65536 / sustained * 1e9 * 1024 / 1e12, 1)
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
    out["note"] = ("the exact fp32 scale-accumulate needs 32 VALU instructions per MFMA; with two or more waves per SIMD "
                   "the times of the two pipes add (in cycles, not through a clock drop), also when they come from "
                   "separate waves: the ceilings are what any kernel with these semantics can reach at 4 waves per SIMD; "
                   "the last one is the same instruction stream at the lower clock the part sustains when operands change "
                   "as they do on real tensors (still from registers: no LDS or memory traffic)")
    return out


def timed_us(torch, fn, n, warm=3):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(n):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / n


def other_configurations(jf, torch):
    """Absolute TOP/s and fraction of the dense INT8 peak for the two other GEMM configurations: the GPT-2 small linear
    set (12288 tokens; forward, dgrad with stochastic rounding, wgrad) and the 8192^3 stress GEMM with requantised
    output in deterministic and stochastic mode (synthetic data of the configurations' distributions, fp32 scales)."""
    out = {}
    g = torch.Generator().manual_seed(0)
    T = 12288
    layers = []
    for name, cin, cout in (("qkv", 768, 2304), ("proj", 768, 768), ("fc", 768, 3072), ("fc2", 3072, 768)):
        qx, sx = jf.quantize(torch.randn(T, cin, generator=g).cuda(), scale_dtype=torch.float32)
        qw, sw = jf.quantize((torch.randn(cout, cin, generator=g) * 0.02).cuda(), scale_dtype=torch.float32)
        qg, sg = jf.quantize((torch.randn(T, cout, generator=g) * 1e-3).cuda(), jf.ROUND_STOCHASTIC, torch.float32, seed=0, offset=0)
        layers.append((name, cin, cout, qx, sx, qw, sw, qg, sg))

    def small_step():
        for name, cin, cout, qx, sx, qw, sw, qg, sg in layers:
            jf.igemm_block_q(qx, qw, sx.t(), sw.t(), jf.B_NK)
            jf.igemm_block_q(qg, qw, sg.t(), sw, jf.B_KN, rounding=jf.ROUND_STOCHASTIC, seed=1, offset=0)
            jf.igemm_block_fp(qg, qx, sg, sx, jf.B_KN, torch.float16, a_layout=jf.A_KM, splitk=0)
    us = timed_us(torch, small_step, 50)
    nops = sum(3 * 2.0 * T * cin * cout for _, cin, cout, *_ in layers)
    out["gpt2_small_set_12288_tokens"] = {"us_per_set": round(us, 1), "TOP/s": round(nops / us / 1e6, 1),
                                          "frac_of_int8_peak": round(nops / us / 1e6 / INT8_PEAK_TOPS, 4),
                                          "wgrad": "gradient read in place, library K split"}
    del layers
    n = 8192
    a = torch.randn(n, n, generator=g) / torch.sqrt(torch.randn(3, n, n, generator=g).pow_(2).mean(0))   # Student-t, 3 dof
    qa, sa = jf.quantize(a.cuda(), scale_dtype=torch.float32)
    del a
    qb, sb = jf.quantize((torch.randn(n, n, generator=g) * 0.02).cuda(), scale_dtype=torch.float32)
    for key, kw in (("deterministic", {}), ("stochastic", dict(rounding=jf.ROUND_STOCHASTIC, seed=5, offset=11))):
        us = timed_us(torch, lambda: jf.igemm_block_q(qa, qb, sa.t(), sb.t(), jf.B_NK, **kw), 30)
        out[f"stress_8192_cubed_{key}"] = {"us": round(us, 1), "TOP/s": round(2.0 * n ** 3 / us / 1e6, 1),
                                           "frac_of_int8_peak": round(2.0 * n ** 3 / us / 1e6 / INT8_PEAK_TOPS, 4)}
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


def _torch_emulation(torch, A8, B8_nk, sa_km, sb_km):
    """The PyTorch emulation of the per-block linear forward on the host: per 32-deep K block an exact fp32 matmul of
    the INT8 codes (32 * 127^2 < 2^24), scaled by the outer product of the two block-scale vectors, accumulated in
    ascending K-block order; then absmax per 32x32 output block, q = clamp(round(127 * acc / amax)).  A8 [M,K] int8,
    B8_nk [N,K] int8, sa_km [K/32, M/32], sb_km [K/32, N/32] fp32.  Returns (codes int8 [M,N], scales fp32)."""
    M, K = A8.shape
    N = B8_nk.shape[0]
    acc = torch.zeros(M, N, dtype=torch.float32)
    for kb in range(K // 32):
        d = A8[:, kb * 32:(kb + 1) * 32].float() @ B8_nk[:, kb * 32:(kb + 1) * 32].float().t()
        sab = sa_km[kb].repeat_interleave(32)[:, None] * sb_km[kb].repeat_interleave(32)[None, :]
        acc += sab * d
    blocks = acc.view(M // 32, 32, N // 32, 32)
    amax = blocks.abs().amax(dim=(1, 3), keepdim=True)
    q = torch.where(amax > 0, torch.round(127.0 * blocks / amax), torch.zeros(())).clamp_(-127, 127)
    return q.to(torch.int8).view(M, N), (amax / 127.0).view(M // 32, N // 32)


def cpu_baseline(ops, rows):
    """The CPU path beside the GPU numbers, on this host's cores.  `value`: the PyTorch emulation (all torch threads) on
    the four forward GEMMs of the timed step restricted to their first `rows` token rows (a bounded sample of the workload).
    Next to it: the same emulation on the 2048 x 768 x 768 seed-0 case (median of 3) with the number of INT8 codes in
    which it differs from the canonical fused arithmetic (a separate multiply and add round differently from an fma),
    and the C restatement under oracle/ (OpenMP) timed on the same two inputs."""
    import platform
    import statistics
    import numpy as np
    import torch
    from oracle import oracle as O
    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    O.set_threads(threads)
    model = platform.processor() or ""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    cpu = lambda t: t.cpu().contiguous()
    nops, dt, dt_oracle = 0.0, 0.0, 0.0
    for o in ops:                                                  # the four forward GEMMs of the timed step
        qx, qw, sxT, swT = cpu(o["qx"][:rows]), cpu(o["qw"]), cpu(o["sxT"][:, : rows // 32]), cpu(o["swT"])
        nops += 2.0 * rows * o["cin"] * o["cout"]
        t0 = time.perf_counter()
        _torch_emulation(torch, qx, qw, sxT, swT)
        dt += time.perf_counter() - t0
        t0 = time.perf_counter()
        O.igemm_block_q(qx.numpy(), qw.numpy(), sxT.numpy(), swT.numpy(), 0)
        dt_oracle += time.perf_counter() - t0
    out = {"value": round(nops / dt / 1e12, 5), "unit": "TOP/s", "cores": threads, "kind": "port",
           "sample": f"PyTorch emulation of the four forward GEMMs of the step (qkv, proj, fc, fc2), first {rows} of 8192 "
                     f"token rows, {nops:.3g} of the step's 1.51e12 ops in {dt:.1f} s, 1 run",
           "cpu_model": model, "torch_version": torch.__version__,
           "c_restatement_same_sample": {"TOP/s": round(nops / dt_oracle / 1e12, 5), "seconds": round(dt_oracle, 2), "threads": threads}}
    # the 2048 x 768 x 768 case, seed 0
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2048, 768, generator=g)
    w = torch.randn(768, 768, generator=g) * 0.02
    qx1, sx1 = O.quantize(x.numpy())
    qw1, sw1 = O.quantize(w.numpy())
    sx1T, sw1T = np.ascontiguousarray(sx1.T), np.ascontiguousarray(sw1.T)
    tx = [torch.from_numpy(a) for a in (qx1, qw1, sx1T, sw1T)]
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        eq, es = _torch_emulation(torch, *tx)
        times.append(time.perf_counter() - t0)
    t0 = time.perf_counter()
    wq, ws = O.igemm_block_q(qx1, qw1, sx1T, sw1T, 0)
    dt_oracle = time.perf_counter() - t0
    uq, _ = O.requant(O.igemm_block_f32(qx1, qw1, sx1T, sw1T, 0, fused=False))
    med = statistics.median(times)
    out["case_2048x768x768_seed0"] = {
        "emulation_ms_median_of_3": round(med * 1e3, 1), "emulation_TOP/s": round(2.0 * 2048 * 768 * 768 / med / 1e12, 5),
        "c_restatement_ms": round(dt_oracle * 1e3, 1), "codes": int(wq.size),
        "codes_emulation_differs_from_fused": int((eq.numpy() != wq).sum()),
        "codes_unfused_restatement_differs_from_fused": int((uq != wq).sum())}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--cpu-rows", type=int, default=8192, help="token rows of the fc forward GEMM the CPU baseline runs")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--pmc-probe", action="store_true", help="copy kernel + 3 GEMM launches only (for rocprofv3 --pmc)")
    ap.add_argument("--roofline-only", action="store_true", help="only the dominant-kernel measurement (for rocprofv3 --stats)")
    ap.add_argument("--extras-only", action="store_true", help="only the block-kernel section (for rocprofv3 --pmc)")
    ap.add_argument("--calibration-only", action="store_true", help="only the register-only calibration loops")
    ap.add_argument("--block-only", action="store_true", help="only the transformer-block comparison")
    ap.add_argument("--stack-only", choices=["int8", "bf16"], default=None,
                    help="10 steps of a three-block GPT-2 XL stack through the INT8 recipe or plain torch bf16 (for rocprofv3 --stats)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (--gpus 1); nothing here uses a second GPU")

    import torch
    import jetfire_hip as jf
    jf.lib()
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    torch.cuda.set_device(0)
    if a.calibration_only:
        print(json.dumps({"calibration": calibration(jf, torch)}))
        return
    if a.block_only:
        print(json.dumps({"xl_block_forward_backward": recipe_block(torch),
                          "gpt2_small_block_forward_backward": recipe_block(torch, shape=(12, 1024, 768, 12)),
                          "host_call_overhead": host_call_overhead(jf, torch)}))
        return
    if a.stack_only:
        print(json.dumps({"stack_of_3_blocks_ms": recipe_block(torch, only=a.stack_only)}))
        return
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
    # the clocks of this part settle only after a few tenths of a second of sustained load (see dominant_kernel_roofline):
    # untimed steps go on until the GPU has been busy for 0.4 s, whatever --warmup says
    t_warm, extra = time.perf_counter(), 0
    while time.perf_counter() - t_warm < 0.4:
        for i in range(20):
            step(jf, torch, ops, a.warmup + a.steps + extra + i)
        extra += 20
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
        "untimed_steps": a.warmup + extra, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 (int32 block accumulate, fp32 scale-accumulate)", "data": "synthetic",
        "config": {"workload": "GPT-2 XL linear set, 8192 tokens: {qkv 1600->4800, proj 1600->1600, fc 1600->6400, "
                               "fc2 6400->1600} x {forward (requantised), dgrad (stochastic), wgrad (fp16)}, "
                               "32x32 per-block INT8, fp32 scales, 1% outlier channels x20",
                   "ops_per_step": step_ops(), "pct_of_int8_peak": round(100 * tops / INT8_PEAK_TOPS, 2),
                   "event_ms_per_step": round(e0.elapsed_time(e1) / a.steps, 4)},
        "roofline": roof,
    }
    if not a.no_extras:
        out["calibration"] = cal = calibration(jf, torch)
        # the dominant kernel against what any kernel with these semantics can reach (the register-only K-block stream at
        # the clock it sustains on changing operands, and, in cycles, at an unchanged clock)
        roof["frac_of_calibrated_ceiling"] = round(roof["achieved"] / cal["ceiling_TOPs_k_block_stream_changing_operands"], 3)
        stream_cycles = [r["cycles"] for r in cal["rows"] if r["case"] == "gemm_k_block_stream" and r["waves_per_simd"] == 4]
        if stream_cycles:
            roof["frac_of_calibrated_ceiling_in_cycles"] = round(stream_cycles[0] / roof["phases"]["simd_cycles_per_block_product"], 3)
        out["other_configurations"] = other_configurations(jf, torch)
        out["memory_bound_kernels"] = nonlinear_extras(jf, torch)
        out["deep_k_weight_gradients"] = deep_k_weight_gradients(jf, torch)
        out["fc_forward_with_gelu"] = fused_fc_gelu(jf, torch, ops)
        out["fc2_dgrad_with_gelu_backward"] = fused_fc2_dgrad_gelu_bwd(jf, torch, ops)
        out["xl_block_forward_backward"] = recipe_block(torch)
        out["gpt2_small_block_forward_backward"] = recipe_block(torch, shape=(12, 1024, 768, 12))
        out["host_call_overhead"] = host_call_overhead(jf, torch)
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline(ops, a.cpu_rows)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
