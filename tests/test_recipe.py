"""End-to-end check of the operator sequence of the INT8 GPT-2 recipe (our counterpart of the autograd
Functions of INT8_GPT2/qmodel.py) against an fp32 torch transformer block: outputs and gradients agree within
quantisation noise, and a small stack trains."""
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


def ref_block(x, blk):
    C = x.shape[-1]
    B, T, _ = x.shape
    h = F.layer_norm(x, (C,), blk.ln_1, None, 0.0)
    qkv = F.linear(h, blk.w_qkv, blk.b_qkv)
    q, k, v = (t.view(B, T, blk.n_head, C // blk.n_head).transpose(1, 2) for t in qkv.split(C, dim=2))
    y = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).contiguous().view(B, T, C)
    x = x + F.linear(y, blk.w_attn_proj, blk.b_attn_proj)
    h = F.layer_norm(x, (C,), blk.ln_2, None, 0.0)
    return x + F.linear(F.gelu(F.linear(h, blk.w_fc, blk.b_fc)), blk.w_mlp_proj, blk.b_mlp_proj)


def cos(a, b):
    return float(F.cosine_similarity(a.detach().reshape(-1).float(), b.detach().reshape(-1).float(), dim=0))


def test_one_block_matches_fp32_reference():
    from recipe import QStack
    torch.manual_seed(0)
    B, T, C, H = 2, 64, 128, 4
    model = QStack(1, C, H).cuda()
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() == 1:
                p.add_(0.1 * torch.randn_like(p))
    x = torch.randn(B, T, C, device="cuda", requires_grad=True)
    w = torch.randn(B, T, C, device="cuda")
    out = model(x)
    assert out.shape == x.shape and out.dtype == torch.float32
    (out * w).sum().backward()
    got = {n: p.grad.clone() for n, p in model.named_parameters()}
    gx = x.grad.clone()
    for p in model.parameters():
        p.grad = None
    x2 = x.detach().clone().requires_grad_(True)
    ref = ref_block(x2, model.blocks[0])
    (ref * w).sum().backward()
    assert cos(out, ref) > 0.999
    assert cos(gx, x2.grad) > 0.99
    for n, p in model.named_parameters():
        assert got[n].shape == p.shape and got[n].dtype == p.dtype
        assert cos(got[n], p.grad) > 0.97, n


def test_block_with_linear_biases_matches_fp32_reference():
    """QBlock(bias=True): the four biases enter in the GEMM epilogues and their gradients are the column sums of the
    layers' quantised output gradients; against the fp32 block with the same biases."""
    from recipe import QStack
    torch.manual_seed(4)
    B, T, C, H = 2, 128, 256, 4
    model = QStack(1, C, H, bias=True).cuda()
    names = [n for n, _ in model.named_parameters()]
    assert sum(".b_" in n for n in names) == 4
    with torch.no_grad():
        for n, p in model.named_parameters():
            if p.dim() == 1:
                p.add_((0.3 if ".b_" in n else 0.1) * torch.randn_like(p))
    x = torch.randn(B, T, C, device="cuda", requires_grad=True)
    w = torch.randn(B, T, C, device="cuda")
    out = model(x)
    (out * w).sum().backward()
    got = {n: p.grad.clone() for n, p in model.named_parameters()}
    gx = x.grad.clone()
    for p in model.parameters():
        p.grad = None
    x2 = x.detach().clone().requires_grad_(True)
    ref = ref_block(x2, model.blocks[0])
    (ref * w).sum().backward()
    assert cos(out, ref) > 0.999
    assert cos(gx, x2.grad) > 0.99
    for n, p in model.named_parameters():
        assert got[n].shape == p.shape and got[n].dtype == p.dtype
        assert cos(got[n], p.grad) > (0.99 if ".b_" in n else 0.97), (n, cos(got[n], p.grad))
    # without the biases the output differs: they are really applied
    with torch.no_grad():
        saved = [p.clone() for n, p in model.named_parameters() if ".b_" in n]
        for n, p in model.named_parameters():
            if ".b_" in n:
                p.zero_()
        assert cos(model(x), ref) < 0.999
        for (n, p), v in zip([(n, p) for n, p in model.named_parameters() if ".b_" in n], saved):
            p.copy_(v)
        assert torch.equal(model(x), out)                          # cached bias operands follow the parameter's version


def test_xl_width_block_matches_fp32_reference():
    """One block at the GPT-2 XL widths (1600 / 4800 / 6400, 25 heads) on 2048 tokens: every operator at its real
    row length (LayerNorm rows of 50 blocks, GELU rows of 200), weight gradients through the K split."""
    from recipe import QStack
    torch.manual_seed(3)
    B, T, C, H = 2, 1024, 1600, 25
    model = QStack(1, C, H).cuda()
    x = torch.randn(B, T, C, device="cuda", requires_grad=True)
    w = torch.randn(B, T, C, device="cuda")
    out = model(x)
    (out * w).sum().backward()
    got = {n: p.grad.clone() for n, p in model.named_parameters()}
    gx = x.grad.clone()
    for p in model.parameters():
        p.grad = None
    x2 = x.detach().clone().requires_grad_(True)
    ref = ref_block(x2, model.blocks[0])
    (ref * w).sum().backward()
    assert torch.isfinite(out).all() and cos(out, ref) > 0.999
    assert cos(gx, x2.grad) > 0.99
    for n, p in model.named_parameters():
        assert torch.isfinite(got[n]).all() and cos(got[n], p.grad) > 0.97, (n, cos(got[n], p.grad))


def test_twelve_layer_stack_matches_fp32_reference():
    """Twelve blocks (the depth of GPT-2 small; the reference stacks n_layer blocks, INT8_GPT2/qmodel.py:418-446):
    forward output after every depth and the gradients of every layer's weights against the same stack in fp32.
    Quantisation noise grows through the depth (each block requantises its residual stream, every backward GEMM rounds
    stochastically), so the thresholds are per depth (measured: forward 0.99995 at depth 12, weight gradients 0.9988
    and better at every depth); a wrong operand, scale or layout anywhere in the chain fails them by far."""
    from recipe import QStack
    torch.manual_seed(7)
    L, B, T, C, H = 12, 2, 128, 256, 4
    model = QStack(L, C, H).cuda()
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() == 1:
                p.add_(0.1 * torch.randn_like(p))
    x = torch.randn(B, T, C, device="cuda", requires_grad=True)
    w = torch.randn(B, T, C, device="cuda")
    # forward at every depth: a prefix of the stack is a stack
    x_ref = x.detach()
    depth_cos = []
    for d in range(1, L + 1):
        x_ref = ref_block(x_ref, model.blocks[d - 1])
        prefix = QStack(0, C, H)
        prefix.blocks = model.blocks[:d]
        with torch.no_grad():
            depth_cos.append(cos(prefix(x.detach()), x_ref))
    print("forward cosine per depth:", [round(c, 5) for c in depth_cos], flush=True)
    for d, c in enumerate(depth_cos, 1):
        assert c > 0.9999 - 1e-5 * d, (d, c)
    # backward through all twelve
    out = model(x)
    (out * w).sum().backward()
    got = {n: p.grad.clone() for n, p in model.named_parameters()}
    gx = x.grad.clone()
    for p in model.parameters():
        p.grad = None
    x2 = x.detach().clone().requires_grad_(True)
    h = x2
    for blk in model.blocks:
        h = ref_block(h, blk)
    (h * w).sum().backward()
    print("output / input-gradient cosine:", round(cos(out, h), 5), round(cos(gx, x2.grad), 5), flush=True)
    assert cos(out, h) > 0.9998
    assert cos(gx, x2.grad) > 0.99, cos(gx, x2.grad)
    worst = {}
    for n, p in model.named_parameters():
        layer = int(n.split(".")[1])
        c = cos(got[n], p.grad)
        worst[layer] = min(worst.get(layer, 1.0), c)
        assert torch.isfinite(got[n]).all()
    print("worst weight-gradient cosine per layer:", {k: round(v, 4) for k, v in sorted(worst.items())}, flush=True)
    for layer, c in worst.items():
        # the gradient reaching layer l has passed through L-1-l quantised backward blocks
        assert c > 0.997 - 0.0003 * (L - 1 - layer), (layer, c)


def test_bfloat16_stream_between_blocks():
    """The reference casts the fp sum that leaves a block to bfloat16 (qmodel.py:228); here the add kernels write it (and
    the gradient that flows back into a bfloat16 residual) in that type.  Input and its gradient keep float32; the INT8
    stream is quantised from the float32 sums, so the result is as close to the fp32 stack as with a float32 stream up to
    the rounding of the residual."""
    from recipe import QStack
    torch.manual_seed(11)
    L, B, T, C, H = 3, 2, 128, 256, 4
    model = QStack(L, C, H, stream_dtype=torch.bfloat16).cuda()
    x = torch.randn(B, T, C, device="cuda", requires_grad=True)
    w = torch.randn(B, T, C, device="cuda")
    out = model(x)
    assert out.dtype == torch.bfloat16
    out.backward(w.to(torch.bfloat16))
    assert x.grad.dtype == torch.float32
    got = {n: p.grad.clone() for n, p in model.named_parameters()}
    gx = x.grad.clone()
    for p in model.parameters():
        p.grad = None
    x2 = x.detach().clone().requires_grad_(True)
    h = x2
    for blk in model.blocks:
        h = ref_block(h, blk)
    (h * w).sum().backward()
    print("bf16 stream: output / input-gradient cosine:", round(cos(out, h), 5), round(cos(gx, x2.grad), 5), flush=True)
    assert cos(out, h) > 0.9995
    assert cos(gx, x2.grad) > 0.99
    for n, p in model.named_parameters():
        assert got[n].dtype == p.dtype and torch.isfinite(got[n]).all()
        assert cos(got[n], p.grad) > 0.99, (n, cos(got[n], p.grad))


def test_merged_node_equals_the_two_functions():
    """AttentionOutMLP is AttentionOut followed by MLPResidual: same kernels in the same order, so with the same noise
    offsets the outputs and every gradient are the same bits."""
    import recipe
    torch.manual_seed(5)
    B, T, C = 2, 64, 128
    blk = recipe.QBlock(C, 4).cuda()
    res = torch.randn(B, T, C, device="cuda")
    y = torch.randn(B, T, C, device="cuda").half()
    gout = torch.randn(B, T, C, device="cuda")

    def run(merged):
        torch.manual_seed(123)                                    # rewinds the stochastic-rounding stream
        r, yy = res.clone().requires_grad_(True), y.clone().requires_grad_(True)
        for p in blk.parameters():
            p.grad = None
        if merged:
            fp, q, s, m, rs = recipe.AttentionOutMLP.apply(r, yy, blk.w_attn_proj, blk.w_fc, blk.w_mlp_proj, blk.ln_2, torch.float32)
        else:
            a = recipe.AttentionOut.apply(r, yy, blk.w_attn_proj)
            fp, q, s, m, rs = recipe.MLPResidual.apply(*a[:3], blk.w_fc, blk.w_mlp_proj, blk.ln_2, a[3], a[4])
        out = recipe.StreamEnd.apply(fp, q, s)
        out.backward(gout)
        return [fp.detach(), q.view(torch.int8), s, m, rs, r.grad, yy.grad, blk.w_attn_proj.grad, blk.w_fc.grad,
                blk.w_mlp_proj.grad, blk.ln_2.grad]
    for i, (a, b) in enumerate(zip(run(True), run(False))):
        assert torch.equal(a, b), i


def test_small_stack_trains():
    from recipe import QStack
    torch.manual_seed(1)
    B, T, C, H = 2, 64, 128, 4
    model = QStack(2, C, H).cuda()
    opt = torch.optim.AdamW(model.parameters(), lr=3e-3)
    x = torch.randn(B, T, C, device="cuda")
    target = torch.roll(x, 1, dims=1) * 0.5 + 0.1
    losses = []
    for _ in range(20):
        opt.zero_grad(set_to_none=True)
        loss = F.mse_loss(model(x), target)
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert losses[-1] < 0.8 * losses[0], losses
    assert all(torch.isfinite(p).all() for p in model.parameters())


def test_weight_codes_are_cached_per_weight_version():
    """A weight is quantised once per value: repeated forwards reuse its codes, an optimizer-style in-place update
    re-quantises it, and cached codes are the ones a fresh quantisation gives."""
    import recipe
    from Nonlinear import int8_quantize
    torch.manual_seed(2)
    model = recipe.QStack(1, 128, 4).cuda()
    x = torch.randn(2, 64, 128, device="cuda")
    recipe.weight_codes.clear()
    recipe.weight_codes.hits = recipe.weight_codes.misses = 0
    with torch.no_grad():
        y0 = model(x)
        assert (recipe.weight_codes.misses, recipe.weight_codes.hits) == (4, 0)
        y1 = model(x)
        assert (recipe.weight_codes.misses, recipe.weight_codes.hits) == (4, 4)
        assert torch.equal(y0, y1)
        w = model.blocks[0].w_fc
        q, s = recipe.weight_codes.get(w)
        q2, s2 = int8_quantize(w.detach(), 32)
        assert torch.equal(q, q2) and torch.equal(s, s2)
        w.mul_(2.0)                                               # what an optimizer step does: in place, new version
        q3, s3 = recipe.weight_codes.get(w)
        assert recipe.weight_codes.misses == 5
        assert torch.equal(q3, q) and not torch.equal(s3, s)      # same codes (exact rescale by 2), doubled scales
        y2 = model(x)
        assert not torch.equal(y2, y1)
    del model, w
    import gc
    gc.collect()
    assert len(recipe.weight_codes._entries) == 0
