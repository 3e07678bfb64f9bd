"""GPU parity of the DiT Block (HIP attention path + library GEMMs + torch elementwise rules) and of its forward-mode
tangent against the CPU oracle of the block (torch fp32 under torch.func.jvp, pinned in tests/test_oracle_dit_block.py)
on the same 16-bit weights and inputs.

Tolerance: a block chains about ten 16-bit stages; outputs are compared with relative-L2 <= 1e-2 and
max-abs <= 3e-2 * max(1, max|want|).  The residual stream dominates `out`, so the same bar is also applied to
`out - x` (the part the block computes) with relative-L2 <= 2e-2.
"""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def check(oracle, name, got, want, rel_l2=1e-2, max_abs=3e-2):
    ma, rl = oracle.error_metrics(got.float().cpu(), want)
    lim = max_abs * max(1.0, float(want.abs().max()))
    print(f"  {name}: max_abs={ma:.3e} (limit {lim:.3e}) rel_l2={rl:.3e}", flush=True)
    assert math.isfinite(ma) and ma <= lim, f"{name}: max-abs {ma} > {lim}"
    assert rl <= rel_l2, f"{name}: rel-L2 {rl} > {rel_l2}"


def build(pkg, gpu, D, Kc, H, lora_dim, dtype, seed):
    torch.manual_seed(seed)
    m = pkg.Block(D, Kc, H, use_adaln_lora=bool(lora_dim), adaln_lora_dim=lora_dim or 256)
    m.init_weights()
    with torch.no_grad():    # the reference starts the last modulation layer at zero (identity block): make it do something
        for mod in (m.adaln_modulation_self_attn, m.adaln_modulation_cross_attn, m.adaln_modulation_mlp):
            last = mod[-1].weight
            last.copy_(torch.randn_like(last) / last.shape[1] ** 0.5)
        for att in (m.self_attn, m.cross_attn):
            att.q_norm.weight.add_(0.2 * torch.randn_like(att.q_norm.weight))
            att.k_norm.weight.add_(0.2 * torch.randn_like(att.k_norm.weight))
    return m.to(device=gpu, dtype=dtype).eval()


def run(pkg, oracle, nr_oracle, block_oracle, gpu, B, T, Hh, W, D, H, Mk, Kc, lora_dim=0, dtype=torch.bfloat16, seed=0):
    print(f"block case B={B} T={T} H={Hh} W={W} D={D} heads={H} Mk={Mk} Kc={Kc} lora={lora_dim} {dtype} seed={seed}", flush=True)
    m = build(pkg, gpu, D, Kc, H, lora_dim, dtype, seed)
    g = torch.Generator().manual_seed(seed + 1)
    r = lambda *s: torch.randn(*s, generator=g)
    x, tx = r(B, T, Hh, W, D).to(dtype), (0.3 * r(B, T, Hh, W, D)).to(dtype)
    emb, temb = r(B, T, D).to(dtype), (0.3 * r(B, T, D)).to(dtype)
    ctx = r(B, Mk, Kc).to(dtype)
    lora = (0.3 * r(B, T, 3 * D)).to(dtype) if lora_dim else None
    tlora = (0.1 * r(B, T, 3 * D)).to(dtype) if lora_dim else None
    hd = D // H
    angles = torch.from_numpy(nr_oracle.rope_angles_3d(T, Hh, W, hd))
    rope = angles.reshape(-1, 1, 1, hd).to(gpu)
    d = lambda t: None if t is None else t.to(gpu)
    with torch.no_grad():
        out = m(d(x), d(emb), d(ctx), rope, d(lora))
    out2, tout = m.forward_jvp(d(x), d(tx), d(emb), d(temb), d(ctx), rope, d(lora), d(tlora))
    torch.cuda.synchronize()
    assert out.shape == x.shape and out.dtype == dtype and tout.shape == x.shape
    want, twant = block_oracle.block_torch(m.state_dict(), x, emb, ctx, angles.numpy(), H, lora, tx, temb, tlora)
    check(oracle, "out", out, want)
    check(oracle, "out (jvp call)", out2, want)
    check(oracle, "tout", tout, twant)
    check(oracle, "out - x", out.float().cpu() - x.float(), want - x.float(), rel_l2=2e-2)
    check(oracle, "tout - tx", tout.float().cpu() - tx.float(), twant - tx.float(), rel_l2=2e-2)


@pytest.mark.parametrize("lora_dim", [0, 16])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_block_small(pkg, oracle, nr_oracle, block_oracle, gpu, lora_dim, dtype):
    run(pkg, oracle, nr_oracle, block_oracle, gpu, B=2, T=2, Hh=4, W=6, D=256, H=2, Mk=20, Kc=96, lora_dim=lora_dim, dtype=dtype, seed=lora_dim)


def test_block_2b_widths_reduced_length(pkg, oracle, nr_oracle, block_oracle, gpu):
    """The 2B DiT's block (2048 wide, 16 heads of 128, text context 1024 wide x 512 tokens, adaLN-LoRA 256) on a
    3 x 8 x 16 token grid."""
    run(pkg, oracle, nr_oracle, block_oracle, gpu, B=1, T=3, Hh=8, W=16, D=2048, H=16, Mk=512, Kc=1024, lora_dim=256, seed=3)


def test_block_14b_widths_reduced_length(pkg, oracle, nr_oracle, block_oracle, gpu):
    """The 14B DiT's block (5120 wide, 40 heads of 128, adaLN-LoRA 256) on a 2 x 6 x 8 token grid: LayerNorm rows of 10
    chunks per lane, 40 heads through the RMSNorm + RoPE kernel's head grouping."""
    run(pkg, oracle, nr_oracle, block_oracle, gpu, B=1, T=2, Hh=6, W=8, D=5120, H=40, Mk=64, Kc=1024, lora_dim=256, seed=4)


def test_block_with_image_context(pkg, oracle, nr_oracle, block_oracle, gpu):
    """image_context_dim: the cross-attention also attends to an image context (minimal_v4_dit.py:451-493)."""
    B, T, Hh, W, D, H, Mk, Kc, Mi, Ki = 2, 2, 4, 6, 256, 2, 20, 96, 12, 80
    torch.manual_seed(7)
    m = pkg.Block(D, Kc, H, use_adaln_lora=True, adaln_lora_dim=16, image_context_dim=Ki)
    m.init_weights()
    with torch.no_grad():
        for mod in (m.adaln_modulation_self_attn, m.adaln_modulation_cross_attn, m.adaln_modulation_mlp):
            mod[-1].weight.copy_(torch.randn_like(mod[-1].weight) / 4.0)
    m = m.to(device=gpu, dtype=torch.bfloat16).eval()
    assert "cross_attn.k_img.weight" in m.state_dict() and "cross_attn.k_img_norm.weight" in m.state_dict()
    g = torch.Generator().manual_seed(8)
    r = lambda *s: torch.randn(*s, generator=g)
    x, tx = r(B, T, Hh, W, D).bfloat16(), (0.3 * r(B, T, Hh, W, D)).bfloat16()
    emb, temb, lora = r(B, T, D).bfloat16(), (0.3 * r(B, T, D)).bfloat16(), (0.3 * r(B, T, 3 * D)).bfloat16()
    ctx, img = r(B, Mk, Kc).bfloat16(), r(B, Mi, Ki).bfloat16()
    hd = D // H
    angles = torch.from_numpy(nr_oracle.rope_angles_3d(T, Hh, W, hd))
    rope = angles.reshape(-1, 1, 1, hd).to(gpu)
    d = lambda t: t.to(gpu)
    with torch.no_grad():
        out = m(d(x), d(emb), (d(ctx), d(img)), rope, d(lora))
    out2, tout = m.forward_jvp(d(x), d(tx), d(emb), d(temb), (d(ctx), d(img)), rope, d(lora), None)
    want, twant = block_oracle.block_torch(m.state_dict(), x, emb, (ctx, img), angles.numpy(), H, lora, tx, temb, None)
    check(oracle, "out", out, want)
    check(oracle, "out (jvp call)", out2, want)
    check(oracle, "tout", tout, twant)
    check(oracle, "out - x", out.float().cpu() - x.float(), want - x.float(), rel_l2=2e-2)


def test_inference_path_matches_autograd_path(pkg, oracle, nr_oracle, gpu):
    """Under no_grad the block runs the fused elementwise passes; with autograd it runs tensor-library ops around the same
    kernels.  Same arithmetic up to the 16-bit roundings between the unfused ops."""
    B, T, Hh, W, D, H, Mk, Kc = 1, 2, 4, 8, 256, 2, 24, 96
    m = build(pkg, gpu, D, Kc, H, 16, torch.bfloat16, 21)
    g = torch.Generator().manual_seed(22)
    r = lambda *s: torch.randn(*s, generator=g).bfloat16().to(gpu)
    x, emb, ctx, lora = r(B, T, Hh, W, D), r(B, T, D), r(B, Mk, Kc), 0.3 * r(B, T, 3 * D)
    hd = D // H
    rope = torch.from_numpy(nr_oracle.rope_angles_3d(T, Hh, W, hd)).reshape(-1, 1, 1, hd).to(gpu)
    with torch.no_grad():
        fused = m(x, emb, ctx, rope, lora)
    with torch.enable_grad():
        plain = m(x.clone().requires_grad_(True), emb, ctx, rope, lora)
    check(oracle, "fused vs autograd path", fused, plain.detach().float().cpu(), rel_l2=1e-2)


def test_fresh_block_is_the_identity(pkg, nr_oracle, gpu):
    """minimal_v4_dit.py:1095-1111: after init_weights the gates are zero."""
    torch.manual_seed(0)
    m = pkg.Block(256, 96, 2, use_adaln_lora=True, adaln_lora_dim=16)
    m.init_weights()
    m = m.to(device=gpu, dtype=torch.bfloat16).eval()
    x = torch.randn(1, 2, 4, 4, 256, device=gpu, dtype=torch.bfloat16)
    tx = torch.randn_like(x)
    emb = torch.randn(1, 2, 256, device=gpu, dtype=torch.bfloat16)
    lora = torch.zeros(1, 2, 768, device=gpu, dtype=torch.bfloat16)
    ctx = torch.randn(1, 8, 96, device=gpu, dtype=torch.bfloat16)
    with torch.no_grad():
        out = m(x, emb, ctx, None, lora)
    out2, tout = m.forward_jvp(x, tx, emb, torch.randn_like(emb), ctx, None, lora, None)
    assert torch.equal(out, x) and torch.equal(out2, x) and torch.equal(tout, tx)


def test_block_reverse_mode(pkg, oracle, nr_oracle, gpu):
    """The block's forward is differentiable end to end (torch autograd around the HIP backward kernels): the gradient of
    x against torch autograd of the same block with the attention calls replaced by fp32 math SDPA on the CPU."""
    B, T, Hh, W, D, H, Mk, Kc = 1, 2, 4, 8, 256, 2, 24, 96
    m = build(pkg, gpu, D, Kc, H, 16, torch.bfloat16, 5).train()
    g = torch.Generator().manual_seed(6)
    r = lambda *s: torch.randn(*s, generator=g)
    x, emb, ctx, lora, dout = r(B, T, Hh, W, D).bfloat16(), r(B, T, D).bfloat16(), r(B, Mk, Kc).bfloat16(), (0.3 * r(B, T, 3 * D)).bfloat16(), r(B, T, Hh, W, D).bfloat16()
    hd = D // H
    angles = torch.from_numpy(nr_oracle.rope_angles_3d(T, Hh, W, hd))
    xd = x.to(gpu).requires_grad_(True)
    out = m(xd, emb.to(gpu), ctx.to(gpu), angles.reshape(-1, 1, 1, hd).to(gpu), lora.to(gpu))
    out.backward(dout.to(gpu))
    torch.cuda.synchronize()
    # oracle: reverse mode of the block oracle's function in fp32
    import __graft_entry__ as entry
    bo = entry.load_dit_block_oracle()
    xr = x.float().requires_grad_(True)
    want_out, _ = bo.block_torch(m.state_dict(), xr, emb, ctx, angles.numpy(), H, lora, keep_graph_input=xr)
    (want_dx,) = torch.autograd.grad(want_out, xr, grad_outputs=dout.float())
    check(oracle, "dx", xd.grad, want_dx)
    for name, prm in m.named_parameters():
        assert prm.grad is not None and torch.isfinite(prm.grad.float()).all(), name


def test_block_with_image_context_reverse_mode(pkg, oracle, nr_oracle, block_oracle, gpu):
    """Reverse mode through the image-conditioned cross-attention (two attention calls summed): the gradient of x
    against torch autograd of the block oracle."""
    B, T, Hh, W, D, H, Mk, Kc, Mi, Ki = 1, 2, 4, 6, 256, 2, 20, 96, 12, 80
    torch.manual_seed(9)
    m = pkg.Block(D, Kc, H, use_adaln_lora=True, adaln_lora_dim=16, image_context_dim=Ki)
    m.init_weights()
    with torch.no_grad():
        for mod in (m.adaln_modulation_self_attn, m.adaln_modulation_cross_attn, m.adaln_modulation_mlp):
            mod[-1].weight.copy_(torch.randn_like(mod[-1].weight) / 4.0)
    m = m.to(device=gpu, dtype=torch.bfloat16).train()
    g = torch.Generator().manual_seed(10)
    r = lambda *s: torch.randn(*s, generator=g)
    x, emb, lora = r(B, T, Hh, W, D).bfloat16(), r(B, T, D).bfloat16(), (0.3 * r(B, T, 3 * D)).bfloat16()
    ctx, img, dout = r(B, Mk, Kc).bfloat16(), r(B, Mi, Ki).bfloat16(), r(B, T, Hh, W, D).bfloat16()
    hd = D // H
    angles = torch.from_numpy(nr_oracle.rope_angles_3d(T, Hh, W, hd))
    xd = x.to(gpu).requires_grad_(True)
    out = m(xd, emb.to(gpu), (ctx.to(gpu), img.to(gpu)), angles.reshape(-1, 1, 1, hd).to(gpu), lora.to(gpu))
    out.backward(dout.to(gpu))
    torch.cuda.synchronize()
    xr = x.float().requires_grad_(True)
    want_out, _ = block_oracle.block_torch(m.state_dict(), xr, emb, (ctx, img), angles.numpy(), H, lora, keep_graph_input=xr)
    (want_dx,) = torch.autograd.grad(want_out, xr, grad_outputs=dout.float())
    check(oracle, "out", out.detach(), want_out.detach())
    check(oracle, "dx", xd.grad, want_dx)
    for name, prm in m.named_parameters():
        assert prm.grad is not None and torch.isfinite(prm.grad.float()).all(), name
