"""GPU parity of the DiT network (patch embedding, time embedding, blocks on the HIP kernels, final layer, unpatchify)
and of its forward-mode tangent along (x, timesteps) against the CPU oracle of the network (torch fp32 under
torch.func.jvp, pinned in tests/test_oracle_dit_network.py) on the same 16-bit weights and inputs.

Tolerance: the output is ``linear(layer_norm(...))`` of a stream that went through every block in 16 bits, with no
residual carrying it: relative-L2 <= 2e-2 and max-abs <= 5e-2 * max(1, max|want|), for output and tangent alike;
weight gradients of the whole network (reverse mode through every block) relative-L2 <= 3e-2.
"""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def check(oracle, name, got, want, rel_l2=2e-2, max_abs=5e-2):
    ma, rl = oracle.error_metrics(got.float().cpu(), want)
    lim = max_abs * max(1.0, float(want.abs().max()))
    print(f"  {name}: max_abs={ma:.3e} (limit {lim:.3e}) rel_l2={rl:.3e}", flush=True)
    assert math.isfinite(ma) and ma <= lim, f"{name}: max-abs {ma} > {lim}"
    assert rl <= rel_l2, f"{name}: rel-L2 {rl} > {rel_l2}"


def build(pkg, gpu, dtype, seed, **kw):
    torch.manual_seed(seed)
    net = pkg.MiniTrainDIT(**kw)
    with torch.no_grad():    # the reference starts every last modulation layer at zero: make them do something
        for blk in net.blocks:
            for mod in (blk.adaln_modulation_self_attn, blk.adaln_modulation_cross_attn, blk.adaln_modulation_mlp):
                mod[-1].weight.copy_(torch.randn_like(mod[-1].weight) / mod[-1].weight.shape[1] ** 0.5)
            for att in (blk.self_attn, blk.cross_attn):
                att.q_norm.weight.add_(0.2 * torch.randn_like(att.q_norm.weight))
                att.k_norm.weight.add_(0.2 * torch.randn_like(att.k_norm.weight))
        last = net.final_layer.adaln_modulation[-1].weight
        last.copy_(torch.randn_like(last) / last.shape[1] ** 0.5)
        net.t_embedding_norm.weight.add_(0.2 * torch.randn_like(net.t_embedding_norm.weight))
    return net.to(device=gpu, dtype=dtype).eval()


def run(pkg, oracle, net_oracle, gpu, *, B, C, T, Hh, W, Mk, Kin, dtype=torch.bfloat16, seed=0, per_frame_time=False, img=None, **kw):
    print(f"network case B={B} C={C} T={T} H={Hh} W={W} Mk={Mk} {dtype} seed={seed} {kw}", flush=True)
    net = build(pkg, gpu, dtype, seed, in_channels=C, **kw)
    p, r, heads = kw["patch_spatial"], kw["patch_temporal"], kw["num_heads"]
    g = torch.Generator().manual_seed(seed + 1)
    rn = lambda *s: torch.randn(*s, generator=g)
    x, tx = rn(B, C, T, Hh, W).to(dtype), (0.3 * rn(B, C, T, Hh, W)).to(dtype)
    Tt = T // r if per_frame_time else 1
    fp32_strategy = kw.get("use_wan_fp32_strategy", False)       # timesteps then arrive in fp32 and the output is fp32
    ts = (torch.rand(B, Tt, generator=g) * 1.4 + 0.05).to(torch.float32 if fp32_strategy else dtype)
    tts = (0.2 * rn(B, Tt)).to(ts.dtype)
    ctx = rn(B, Mk, Kin).to(dtype)
    imgc = None if img is None else rn(B, *img).to(dtype)
    pm = (torch.rand(B, 1, Hh, W, generator=g) > 0.5).to(dtype) if kw.get("concat_padding_mask", True) else None
    fps = torch.full((B,), 16.0)
    d = lambda t: None if t is None else t.to(gpu)
    with torch.no_grad():
        out = net(d(x), d(ts), d(ctx), fps=d(fps), padding_mask=d(pm), img_context_emb=d(imgc))
    out2, tout = net.forward_jvp(d(x), d(tx), d(ts), d(tts), d(ctx), fps=d(fps), padding_mask=d(pm), img_context_emb=d(imgc))
    torch.cuda.synchronize()
    assert out.shape == (B, kw["out_channels"], T, Hh, W) and tout.shape == out.shape
    assert out.dtype == tout.dtype == out2.dtype == (torch.float32 if fp32_strategy else dtype)
    with torch.no_grad():
        angles = net.pos_embedder.generate_embeddings((B, T // r, Hh // p, W // p, 0), fps=d(fps)).reshape(-1, kw["model_channels"] // heads)
    want, twant = net_oracle.network_torch(net.state_dict(), x, ts, ctx, num_heads=heads, patch_spatial=p, patch_temporal=r,
                                           rope_angles=angles.cpu(), padding_mask=pm, img_context_emb=imgc, tx=tx, ttimesteps=tts)
    check(oracle, "out", out, want)
    check(oracle, "out (jvp call)", out2, want)
    check(oracle, "tout", tout, twant)
    return net, (x, tx, ts, tts, ctx, pm, fps)


SMALL = dict(max_img_h=32, max_img_w=32, max_frames=8, out_channels=4, patch_spatial=2, patch_temporal=1, model_channels=256,
             num_blocks=2, num_heads=2, crossattn_emb_channels=96)


@pytest.mark.parametrize("lora_dim", [0, 16])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_network_small(pkg, oracle, net_oracle, gpu, lora_dim, dtype):
    run(pkg, oracle, net_oracle, gpu, B=2, C=4, T=2, Hh=8, W=12, Mk=20, Kin=96, dtype=dtype, seed=lora_dim,
        use_adaln_lora=bool(lora_dim), adaln_lora_dim=lora_dim or 256, **SMALL)


@pytest.mark.parametrize("lora_dim", [0, 16])
def test_network_fp32_strategy(pkg, oracle, net_oracle, gpu, lora_dim):
    """use_wan_fp32_strategy (set by the released rectified-flow configurations): fp32 timesteps, time embedding, modulation
    MLPs and final layer in fp32, fp32 output (minimal_v4_dit.py:967-988, :1131, :1610)."""
    run(pkg, oracle, net_oracle, gpu, B=2, C=4, T=2, Hh=8, W=12, Mk=20, Kin=96, seed=31 + lora_dim, use_wan_fp32_strategy=True,
        use_adaln_lora=bool(lora_dim), adaln_lora_dim=lora_dim or 256, **SMALL)


def test_network_all_options(pkg, oracle, net_oracle, gpu):
    """Per-frame timesteps, learned per-block position term, text-context projection, image context, temporal patches,
    no padding-mask channel."""
    kw = dict(SMALL, patch_temporal=2, extra_per_block_abs_pos_emb=True, use_crossattn_projection=True, crossattn_proj_in_channels=80,
              extra_image_context_dim=48, concat_padding_mask=False, use_adaln_lora=True, adaln_lora_dim=16)
    run(pkg, oracle, net_oracle, gpu, B=1, C=3, T=4, Hh=8, W=8, Mk=20, Kin=80, seed=5, per_frame_time=True, img=(12, 48), **kw)


def test_network_2b_widths_reduced(pkg, oracle, net_oracle, gpu):
    """The 2B DiT's widths (2048 channels, 16 heads of 128, adaLN-LoRA 256, 16 latent channels in and out, 2 x 2 x 1
    patches, text context 1024 wide) with 2 blocks on a 3 x 8 x 16 token grid."""
    kw = dict(max_img_h=240, max_img_w=240, max_frames=128, out_channels=16, patch_spatial=2, patch_temporal=1, model_channels=2048,
              num_blocks=2, num_heads=16, crossattn_emb_channels=1024, use_adaln_lora=True, adaln_lora_dim=256)
    run(pkg, oracle, net_oracle, gpu, B=1, C=16, T=3, Hh=16, W=32, Mk=512, Kin=1024, seed=9, **kw)


def test_tangent_is_linear_in_its_direction_and_time_direction_matters(pkg, oracle, net_oracle, gpu):
    net, (x, tx, ts, tts, ctx, pm, fps) = run(pkg, oracle, net_oracle, gpu, B=1, C=4, T=2, Hh=8, W=8, Mk=20, Kin=96, seed=13,
                                              use_adaln_lora=True, adaln_lora_dim=16, **SMALL)
    d = lambda t: t.to(gpu)
    _, t_x = net.forward_jvp(d(x), d(tx), d(ts), None, d(ctx), fps=d(fps), padding_mask=d(pm))
    _, t_t = net.forward_jvp(d(x), torch.zeros_like(d(tx)), d(ts), d(tts), d(ctx), fps=d(fps), padding_mask=d(pm))
    _, t_both = net.forward_jvp(d(x), d(tx), d(ts), d(tts), d(ctx), fps=d(fps), padding_mask=d(pm))
    assert float(t_t.float().abs().max()) > 1e-3
    check(oracle, "t(x dir) + t(time dir) vs t(both)", t_x.float() + t_t.float(), t_both.float().cpu())


def test_inference_path_matches_autograd_path_and_backward_runs(pkg, oracle, net_oracle, gpu):
    net = build(pkg, gpu, torch.bfloat16, 17, in_channels=4, use_adaln_lora=True, adaln_lora_dim=16, **SMALL).train()
    g = torch.Generator().manual_seed(18)
    rn = lambda *s: torch.randn(*s, generator=g).bfloat16().to(gpu)
    x, ctx = rn(1, 4, 2, 8, 8), rn(1, 20, 96)
    ts = torch.tensor([[0.7]], device=gpu, dtype=torch.bfloat16)
    pm = torch.zeros(1, 1, 8, 8, device=gpu, dtype=torch.bfloat16)
    fps = torch.full((1,), 16.0, device=gpu)
    with torch.no_grad():
        fused = net(x, ts, ctx, fps=fps, padding_mask=pm)
    xg = x.clone().requires_grad_(True)
    plain = net(xg, ts, ctx, fps=fps, padding_mask=pm)
    check(oracle, "fused vs autograd path", fused, plain.detach().float().cpu())
    plain.backward(torch.randn_like(plain))
    torch.cuda.synchronize()
    assert torch.isfinite(xg.grad.float()).all() and float(xg.grad.float().abs().max()) > 0
    for name, prm in net.named_parameters():
        assert prm.grad is not None and torch.isfinite(prm.grad.float()).all(), name


def test_fresh_network_output_does_not_depend_on_time(pkg, gpu):
    """After init_weights every modulation layer is zero; without adaLN-LoRA the blocks are then the identity, the output is
    ``linear(layer_norm(x))`` whatever the time, and the tangent along the time is exactly zero."""
    torch.manual_seed(0)
    net = pkg.MiniTrainDIT(in_channels=4, use_adaln_lora=False, **SMALL).to(device=gpu, dtype=torch.bfloat16).eval()
    x = torch.randn(1, 4, 2, 8, 8, device=gpu, dtype=torch.bfloat16)
    ctx = torch.randn(1, 20, 96, device=gpu, dtype=torch.bfloat16)
    pm = torch.zeros(1, 1, 8, 8, device=gpu, dtype=torch.bfloat16)
    fps = torch.full((1,), 16.0, device=gpu)
    ts = torch.tensor([[0.3]], device=gpu, dtype=torch.bfloat16)
    out, tout = net.forward_jvp(x, torch.zeros_like(x), ts, torch.ones_like(ts), ctx, fps=fps, padding_mask=pm)
    with torch.no_grad():
        a = net(x, ts, ctx, fps=fps, padding_mask=pm)
        b = net(x, 3 * ts, ctx, fps=fps, padding_mask=pm)
    assert torch.equal(out, a) and torch.equal(a, b)
    assert float(tout.float().abs().max()) == 0.0


def test_video_conditioned_network(pkg, oracle, net_oracle, gpu):
    """MinimalV1LVGDiT (minimal_v1_lvg_dit.py:24-62): the condition mask is one more input channel (zeros for an image
    batch) and the timesteps are scaled; checked against the network oracle on the concatenated input."""
    torch.manual_seed(23)
    kw = dict(SMALL, use_adaln_lora=True, adaln_lora_dim=16)
    net = pkg.MinimalV1LVGDiT(in_channels=4, timestep_scale=0.5, **kw)
    assert net.x_embedder.proj[1].weight.shape[1] == (4 + 1 + 1) * 4
    with torch.no_grad():
        for blk in net.blocks:
            for mod in (blk.adaln_modulation_self_attn, blk.adaln_modulation_cross_attn, blk.adaln_modulation_mlp):
                mod[-1].weight.copy_(torch.randn_like(mod[-1].weight) / 4.0)
        net.final_layer.adaln_modulation[-1].weight.copy_(torch.randn_like(net.final_layer.adaln_modulation[-1].weight) / 4.0)
    net = net.to(device=gpu, dtype=torch.bfloat16).eval()
    g = torch.Generator().manual_seed(24)
    rn = lambda *s: torch.randn(*s, generator=g).bfloat16()
    B, C, T, Hh, W = 1, 4, 2, 8, 8
    x, tx, ctx = rn(B, C, T, Hh, W), 0.3 * rn(B, C, T, Hh, W), rn(B, 20, 96)
    ts, tts = torch.tensor([[1.5]]).bfloat16(), torch.tensor([[0.25]]).bfloat16()
    cond = torch.zeros(B, 1, T, Hh, W).bfloat16()
    cond[:, :, :1] = 1
    pm = torch.zeros(B, 1, Hh, W).bfloat16()
    fps = torch.full((B,), 16.0)
    d = lambda t: t.to(gpu)
    with torch.no_grad():
        out = net(d(x), d(ts), d(ctx), d(cond), fps=d(fps), padding_mask=d(pm))
        out_img = net(d(x[:, :, :1]), d(ts), d(ctx), None, fps=None, padding_mask=d(pm), data_type="image")
    out2, tout = net.forward_jvp(d(x), d(tx), d(ts), d(tts), d(ctx), d(cond), fps=d(fps), padding_mask=d(pm))
    with torch.no_grad():
        angles = net.pos_embedder.generate_embeddings((B, T, Hh // 2, W // 2, 0), fps=d(fps)).reshape(-1, 128).cpu()
        angles_img = net.pos_embedder.generate_embeddings((B, 1, Hh // 2, W // 2, 0), fps=None).reshape(-1, 128).cpu()
    run_oracle = lambda x_, tx_, a_: net_oracle.network_torch(net.state_dict(), x_, ts.float() * 0.5, ctx, num_heads=2, patch_spatial=2,
                                                              patch_temporal=1, rope_angles=a_, padding_mask=pm, tx=tx_, ttimesteps=tts.float() * 0.5)
    want, twant = run_oracle(torch.cat([x, cond], 1), torch.cat([tx, torch.zeros_like(cond)], 1), angles)
    check(oracle, "out", out, want)
    check(oracle, "out (jvp call)", out2, want)
    check(oracle, "tout", tout, twant)
    want_img, _ = run_oracle(torch.cat([x[:, :, :1], torch.zeros_like(cond[:, :, :1])], 1), None, angles_img)
    check(oracle, "out (image batch)", out_img, want_img)


def test_consistency_distillation_step(pkg, oracle, net_oracle, gpu):
    """One step of the kind the forward + JVP path exists for: the tangent of the student along (dx, dt) from ``forward_jvp``
    (no autograd: it is a stop-gradient target), then an ordinary forward and backward of
    ``mean((F - stopgrad(F - g))^2)`` with g the normalised tangent.  The gradients of x and of every weight are checked
    against torch autograd of the network oracle (fp32) for the same cotangent."""
    kw = dict(SMALL, use_adaln_lora=True, adaln_lora_dim=16)
    net = build(pkg, gpu, torch.bfloat16, 29, in_channels=4, **kw).train()
    g = torch.Generator().manual_seed(30)
    rn = lambda *s: torch.randn(*s, generator=g).bfloat16()
    B, C, T, Hh, W = 1, 4, 2, 8, 8
    x, direction, ctx = rn(B, C, T, Hh, W), rn(B, C, T, Hh, W), rn(B, 20, 96)
    ts = torch.tensor([[0.8]]).bfloat16()
    pm = torch.zeros(B, 1, Hh, W).bfloat16()
    fps = torch.full((B,), 16.0)
    d = lambda t: t.to(gpu)
    _, tangent = net.forward_jvp(d(x), d(direction), d(ts), torch.ones_like(d(ts)), d(ctx), fps=d(fps), padding_mask=d(pm))
    assert not tangent.requires_grad
    gn = tangent.float() / (tangent.float().norm() + 0.1)
    xg = d(x).requires_grad_(True)
    out = net(xg, d(ts), d(ctx), fps=d(fps), padding_mask=d(pm))
    loss = ((out.float() - (out.detach().float() - gn)) ** 2).mean()
    loss.backward()
    torch.cuda.synchronize()
    assert math.isfinite(loss.item()) and loss.item() > 0
    dout = (2.0 * gn / out.numel()).cpu()       # d loss / d out
    with torch.no_grad():
        angles = net.pos_embedder.generate_embeddings((B, T, Hh // 2, W // 2, 0), fps=d(fps)).reshape(-1, 128).cpu()
    dx, dw = net_oracle.network_grads_torch(net.state_dict(), x, ts, ctx, dout, num_heads=2, patch_spatial=2, patch_temporal=1,
                                            rope_angles=angles, padding_mask=pm)
    scale = 1.0 / float(dx.abs().max())          # gradients of a mean are tiny: compare them rescaled
    check(oracle, "dx", xg.grad.float().cpu() * scale, dx * scale, rel_l2=2e-2, max_abs=5e-2)
    worst = ("", 0.0)
    for name, prm in net.named_parameters():
        assert prm.grad is not None and name in dw, name
        want = dw[name]
        s = 1.0 / max(float(want.abs().max()), 1e-30)
        ma, rl = oracle.error_metrics(prm.grad.float().cpu() * s, want * s)
        worst = max(worst, (name, rl), key=lambda z: z[1])
        assert rl <= 3e-2, f"{name}: rel-L2 {rl}"
    print(f"  weight gradients: worst rel-L2 {worst[1]:.3e} ({worst[0]})", flush=True)


def test_activation_checkpointing_gives_the_same_gradients(pkg, gpu):
    """sac_config (minimal_v4_dit.py:1660-1686): blocks keep their inputs and their attention results and run again in the
    backward pass (without launching the forward attention kernels again); the recomputation is deterministic, so the
    output, the gradient of x and the gradients of the blocks' weights are the bits of the plain run."""
    kw = dict(SMALL, use_adaln_lora=True, adaln_lora_dim=16)
    plain = build(pkg, gpu, torch.bfloat16, 37, in_channels=4, **kw).train()
    ckpt = build(pkg, gpu, torch.bfloat16, 37, in_channels=4, sac_config=dict(mode="predict2_2b_720_aggressive", every_n_blocks=1), **kw).train()
    ckpt.load_state_dict(plain.state_dict())
    assert plain._checkpoint_every == 0 and ckpt._checkpoint_every == 1
    g = torch.Generator().manual_seed(38)
    rn = lambda *s: torch.randn(*s, generator=g).bfloat16().to(gpu)
    x, ctx, dout = rn(1, 4, 2, 8, 8), rn(1, 20, 96), rn(1, 4, 2, 8, 8)
    ts = torch.tensor([[0.7]], device=gpu, dtype=torch.bfloat16)
    pm = torch.zeros(1, 1, 8, 8, device=gpu, dtype=torch.bfloat16)
    fps = torch.full((1,), 16.0, device=gpu)
    grads = []
    for net in (plain, ckpt):
        xg = x.clone().requires_grad_(True)
        out = net(xg, ts, ctx, fps=fps, padding_mask=pm)
        out.backward(dout)
        torch.cuda.synchronize()
        grads.append((out.detach(), xg.grad, {n: p.grad for n, p in net.named_parameters()}))
    (o0, dx0, w0), (o1, dx1, w1) = grads
    assert torch.equal(o0, o1) and torch.equal(dx0, dx1)
    for name in w0:
        assert w1[name] is not None, name
        if name.startswith(("t_embedder.", "t_embedding_norm.")):
            # the time embedding feeds every block: its gradient is a sum over the blocks, which the two runs add up in 16
            # bits in different orders
            a, b = w0[name].float(), w1[name].float()
            assert float((a - b).norm() / a.norm()) <= 1e-2, name
        else:
            assert torch.equal(w0[name], w1[name]), name


def test_activation_checkpointing_with_every_option(pkg, gpu):
    """The block checkpoint with a learned position term, a projected text context and an image context (all of them carry
    gradients into the checkpointed blocks), every second block checkpointed: gradients of all weights as in the plain run."""
    kw = dict(SMALL, patch_temporal=2, extra_per_block_abs_pos_emb=True, use_crossattn_projection=True, crossattn_proj_in_channels=80,
              extra_image_context_dim=48, concat_padding_mask=False, use_adaln_lora=True, adaln_lora_dim=16, num_blocks=3)
    plain = build(pkg, gpu, torch.bfloat16, 41, in_channels=3, **kw).train()
    ckpt = build(pkg, gpu, torch.bfloat16, 41, in_channels=3, sac_config=dict(mode="block_wise", every_n_blocks=2), **kw).train()
    ckpt.load_state_dict(plain.state_dict())
    g = torch.Generator().manual_seed(42)
    rn = lambda *s: torch.randn(*s, generator=g).bfloat16().to(gpu)
    x, ctx, img, dout = rn(1, 3, 4, 8, 8), rn(1, 20, 80), rn(1, 12, 48), rn(1, 4, 4, 8, 8)
    ts = torch.tensor([[0.7, 0.9]], device=gpu, dtype=torch.bfloat16)
    fps = torch.full((1,), 16.0, device=gpu)
    grads = []
    for net in (plain, ckpt):
        out = net(x, ts, ctx, fps=fps, img_context_emb=img)
        out.backward(dout)
        torch.cuda.synchronize()
        grads.append((out.detach(), {n: p.grad for n, p in net.named_parameters()}))
    (o0, w0), (o1, w1) = grads
    assert torch.equal(o0, o1)
    for name in w0:
        assert w0[name] is not None and w1[name] is not None, name
        a, b = w0[name].float(), w1[name].float()
        if name.startswith("blocks."):
            assert torch.equal(a, b), name
        else:       # sums over the blocks, added up in 16 bits in another order
            assert float((a - b).norm() / a.norm().clamp_min(1e-30)) <= 1e-2, name
