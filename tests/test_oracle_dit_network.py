"""Pins for the CPU oracle of the DiT network around the blocks (no GPU): index maps against einops with the
reference's own pattern strings, a stepwise fp64 recomputation (numpy for everything around the blocks, the separately
pinned block oracle for the blocks), central finite differences for the tangent, and the initialisation property."""
import math

import numpy as np
import pytest
import torch
from einops import rearrange

from test_oracle_dit_block import make_block_weights


def make_network_weights(*, C, C_out, D, H, Kc, p, r, n_blocks, lora_dim, mask, extra, lens=(4, 6, 6), seed=0,
                         zero_last=False, zero_final=False, ctx_proj_in=0, img_dim=0):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    w = {}
    cin = (C + 1 if mask else C) * p * p * r
    w["x_embedder.proj.1.weight"] = rn(D, cin) / cin ** 0.5
    w["t_embedder.1.linear_1.weight"] = rn(D, D) / D ** 0.5
    if not lora_dim:
        w["t_embedder.1.linear_1.bias"] = 0.1 * rn(D)
    w["t_embedder.1.linear_2.weight"] = rn(3 * D if lora_dim else D, D) / D ** 0.5
    w["t_embedding_norm.weight"] = 1 + 0.2 * rn(D)
    for i in range(n_blocks):
        bw = make_block_weights(D, Kc, H, lora_dim, seed + 10 + i, zero_last=zero_last)
        if img_dim:
            bw["cross_attn.k_img.weight"] = rn(D, D) / D ** 0.5
            bw["cross_attn.v_img.weight"] = rn(D, D) / D ** 0.5
            bw["cross_attn.k_img_norm.weight"] = 1 + 0.2 * rn(D // H)
        w.update({f"blocks.{i}.{k}": v for k, v in bw.items()})
    w["final_layer.linear.weight"] = rn(p * p * r * C_out, D) / D ** 0.5
    if lora_dim:
        w["final_layer.adaln_modulation.1.weight"] = rn(lora_dim, D) / D ** 0.5
        w["final_layer.adaln_modulation.2.weight"] = torch.zeros(2 * D, lora_dim, dtype=torch.float64) if zero_final else rn(2 * D, lora_dim) / lora_dim ** 0.5
    else:
        w["final_layer.adaln_modulation.1.weight"] = torch.zeros(2 * D, D, dtype=torch.float64) if zero_final else rn(2 * D, D) / D ** 0.5
    if extra:
        for name, n in zip("thw", lens):
            w[f"extra_pos_embedder.pos_emb_{name}"] = rn(n, D) / D ** 0.5
    if ctx_proj_in:
        w["crossattn_proj.0.weight"] = rn(Kc, ctx_proj_in) / ctx_proj_in ** 0.5
        w["crossattn_proj.0.bias"] = 0.1 * rn(Kc)
    if img_dim:
        w["img_context_proj.0.weight"] = rn(D, img_dim) / img_dim ** 0.5
        w["img_context_proj.0.bias"] = 0.1 * rn(D)
    return w


def make_inputs(B, C, T, Hh, W, Tt, Mk, Kin, seed, img=None):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    return dict(x=rn(B, C, T, Hh, W), ts=torch.rand(B, Tt, generator=g, dtype=torch.float64) * 3 + 0.1, ctx=rn(B, Mk, Kin),
                pm=(torch.rand(B, 1, Hh // 2, W // 2, generator=g) > 0.5).double(),
                tx=0.3 * rn(B, C, T, Hh, W), tts=0.2 * rn(B, Tt), img=None if img is None else rn(B, img[0], img[1]))


def test_index_maps_match_einops_with_the_reference_patterns(net_oracle):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 3, 4, 6, 8))
    want = rearrange(x, "b c (t r) (h m) (w n) -> b t h w (c r m n)", r=2, m=2, n=2)
    assert np.array_equal(net_oracle.patchify_loops(x, 2, 2, 2), want)
    y = rng.standard_normal((2, 2, 3, 4, 2 * 2 * 1 * 5))
    want = rearrange(y, "B T H W (p1 p2 t C) -> B C (T t) (H p1) (W p2)", p1=2, p2=2, t=1)
    assert np.array_equal(net_oracle.unpatchify_loops(y, 2, 1, 5), want)
    y = rng.standard_normal((1, 2, 3, 2, 3 * 3 * 2 * 2))
    want = rearrange(y, "B T H W (p1 p2 t C) -> B C (T t) (H p1) (W p2)", p1=3, p2=3, t=2)
    assert np.array_equal(net_oracle.unpatchify_loops(y, 3, 2, 2), want)


def _stepwise(net_oracle, block_oracle, w, i, *, H, p, r, angles, mask, img=None):
    """numpy fp64 for everything around the blocks; the block oracle for the blocks."""
    n = lambda t: t.numpy()
    x = n(i["x"])
    B, C, T, Hh, W = x.shape
    D = w["x_embedder.proj.1.weight"].shape[0]
    if mask:
        pm = n(i["pm"])
        hh, ww = pm.shape[-2:]
        # nearest-neighbour resize: source index floor(dst * src / dst_size)
        rows = (np.arange(Hh) * hh // Hh)
        cols = (np.arange(W) * ww // W)
        big = pm[:, :, rows][:, :, :, cols]
        x = np.concatenate([x, np.broadcast_to(big[:, :, None], (B, 1, T, Hh, W))], axis=1)
    h = net_oracle.patchify_loops(x, r, p, p) @ n(w["x_embedder.proj.1.weight"]).T
    ts = n(i["ts"])
    half = D // 2
    freqs = 10000.0 ** (-np.arange(half) / half)
    ang = ts[..., None] * freqs
    sample = np.concatenate([np.cos(ang), np.sin(ang)], -1)
    z = sample @ n(w["t_embedder.1.linear_1.weight"]).T
    if "t_embedder.1.linear_1.bias" in w:
        z = z + n(w["t_embedder.1.linear_1.bias"])
    mlp = (z / (1 + np.exp(-z))) @ n(w["t_embedder.1.linear_2.weight"]).T
    lora_form = "final_layer.adaln_modulation.2.weight" in w
    emb, lora = (sample, mlp) if lora_form else (mlp, None)
    emb = emb / np.sqrt((emb ** 2).mean(-1, keepdims=True) + 1e-6) * n(w["t_embedding_norm.weight"])
    ctx = n(i["ctx"])
    gelu = lambda t: 0.5 * t * (1 + np.vectorize(math.erf)(t / math.sqrt(2)))
    if "crossattn_proj.0.weight" in w:
        ctx = gelu(ctx @ n(w["crossattn_proj.0.weight"]).T + n(w["crossattn_proj.0.bias"]))
    if img is not None:
        ctx = (ctx, gelu(n(img) @ n(w["img_context_proj.0.weight"]).T + n(w["img_context_proj.0.bias"])))
    extra = 0.0
    if "extra_pos_embedder.pos_emb_h" in w:
        Tp, Hp, Wp = h.shape[1:4]
        e = (n(w["extra_pos_embedder.pos_emb_t"])[:Tp, None, None] + n(w["extra_pos_embedder.pos_emb_h"])[None, :Hp, None]
             + n(w["extra_pos_embedder.pos_emb_w"])[None, None, :Wp])
        nrm = np.sqrt((e ** 2).sum(-1, keepdims=True))
        # vector_norm gives one number per token; alpha = sqrt(#tokens / #elements) = 1 / sqrt(D)
        extra = (e / (1e-6 + nrm * math.sqrt(nrm.size / e.size)))[None]
    n_blocks = 1 + max(int(k.split(".")[1]) for k in w if k.startswith("blocks."))
    for b in range(n_blocks):
        bw = {k[len(f"blocks.{b}."):]: v for k, v in w.items() if k.startswith(f"blocks.{b}.")}
        out, _ = block_oracle.block_torch(bw, torch.from_numpy(h + extra), torch.from_numpy(emb),
                                          tuple(torch.from_numpy(c) for c in ctx) if isinstance(ctx, tuple) else torch.from_numpy(ctx),
                                          angles, H, None if lora is None else torch.from_numpy(lora), dtype=torch.float64)
        h = out.numpy()
    m = (emb / (1 + np.exp(-emb))) @ n(w["final_layer.adaln_modulation.1.weight"]).T
    if lora_form:
        m = m @ n(w["final_layer.adaln_modulation.2.weight"]).T + lora[..., : 2 * D]
    shift, scale = m[..., :D][:, :, None, None], m[..., D:][:, :, None, None]
    mu = h.mean(-1, keepdims=True)
    var = ((h - mu) ** 2).mean(-1, keepdims=True)
    y = ((h - mu) / np.sqrt(var + 1e-6) * (1 + scale) + shift) @ n(w["final_layer.linear.weight"]).T
    C_out = y.shape[-1] // (p * p * r)
    return net_oracle.unpatchify_loops(y, p, r, C_out)


CASES = [
    dict(lora_dim=0, mask=True, extra=False, r=1, Tt=2, ctx_proj_in=0, img_dim=0),
    dict(lora_dim=8, mask=True, extra=True, r=1, Tt=1, ctx_proj_in=20, img_dim=0),
    dict(lora_dim=8, mask=False, extra=False, r=2, Tt=2, ctx_proj_in=0, img_dim=12),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "-".join(f"{k}{v}" for k, v in c.items()))
def test_network_oracle_matches_stepwise_fp64_recomputation(net_oracle, block_oracle, case):
    B, C, C_out, D, H, Kc, p, Mk = 2, 3, 4, 32, 2, 24, 2, 5
    r, Tt = case["r"], case["Tt"]
    T, Hh, W = 2 * r, 4, 6
    w = make_network_weights(C=C, C_out=C_out, D=D, H=H, Kc=Kc, p=p, r=r, n_blocks=2, lora_dim=case["lora_dim"], mask=case["mask"],
                             extra=case["extra"], seed=3, ctx_proj_in=case["ctx_proj_in"], img_dim=case["img_dim"])
    i = make_inputs(B, C, T, Hh, W, Tt, Mk, case["ctx_proj_in"] or Kc, 4, img=(3, case["img_dim"]) if case["img_dim"] else None)
    hd = D // H
    halfang = np.random.default_rng(5).standard_normal(((T // r) * (Hh // p) * (W // p), hd // 2))
    angles = np.concatenate([halfang, halfang], -1)
    out, _ = net_oracle.network_torch(w, i["x"], i["ts"], i["ctx"], num_heads=H, patch_spatial=p, patch_temporal=r, rope_angles=angles,
                                      padding_mask=i["pm"] if case["mask"] else None, img_context_emb=i["img"], dtype=torch.float64)
    want = _stepwise(net_oracle, block_oracle, w, i, H=H, p=p, r=r, angles=angles, mask=case["mask"], img=i["img"])
    assert out.shape == (B, C_out, T, Hh, W)
    np.testing.assert_allclose(out.numpy(), want, rtol=0, atol=1e-10)


@pytest.mark.parametrize("lora_dim", [0, 8])
def test_network_oracle_tangent_matches_central_differences(net_oracle, lora_dim):
    B, C, C_out, D, H, Kc, p, r, Mk = 1, 2, 2, 16, 2, 12, 2, 1, 4
    T, Hh, W = 2, 4, 4
    w = make_network_weights(C=C, C_out=C_out, D=D, H=H, Kc=Kc, p=p, r=r, n_blocks=2, lora_dim=lora_dim, mask=True, extra=True, seed=7)
    i = make_inputs(B, C, T, Hh, W, T, Mk, Kc, 8)
    halfang = np.random.default_rng(9).standard_normal((T * 2 * 2, D // H // 2))
    angles = np.concatenate([halfang, halfang], -1)
    run = lambda x, ts, **kw: net_oracle.network_torch(w, x, ts, i["ctx"], num_heads=H, patch_spatial=p, patch_temporal=r, rope_angles=angles,
                                                       padding_mask=i["pm"], dtype=torch.float64, **kw)
    out, tout = run(i["x"], i["ts"], tx=i["tx"], ttimesteps=i["tts"])
    eps = 1e-6
    fd = (run(i["x"] + eps * i["tx"], i["ts"] + eps * i["tts"])[0] - run(i["x"] - eps * i["tx"], i["ts"] - eps * i["tts"])[0]) / (2 * eps)
    assert torch.allclose(out, run(i["x"], i["ts"])[0], atol=1e-12)
    err = (tout - fd).abs().max().item() / fd.abs().max().item()
    assert err < 1e-6, err
    # the time direction alone is not zero: the tangent really depends on it
    _, t_only = run(i["x"], i["ts"], tx=torch.zeros_like(i["tx"]), ttimesteps=i["tts"])
    assert t_only.abs().max().item() > 1e-3


def test_network_at_initialisation_is_projection_of_layernorm(net_oracle):
    """Last modulation layers zero (the reference's init_weights) and no LoRA: blocks are the identity and the final
    layer is ``linear(layer_norm(x))``, whatever the timestep."""
    B, C, C_out, D, H, Kc, p, r = 1, 2, 3, 16, 2, 12, 2, 1
    T, Hh, W = 1, 4, 4
    w = make_network_weights(C=C, C_out=C_out, D=D, H=H, Kc=Kc, p=p, r=r, n_blocks=2, lora_dim=0, mask=False, extra=False, seed=11,
                             zero_last=True, zero_final=True)
    i = make_inputs(B, C, T, Hh, W, 1, 4, Kc, 12)
    out, tout = net_oracle.network_torch(w, i["x"], i["ts"], i["ctx"], num_heads=H, patch_spatial=p, patch_temporal=r, dtype=torch.float64,
                                         tx=torch.zeros_like(i["tx"]), ttimesteps=i["tts"])
    h = net_oracle.patchify_loops(i["x"].numpy(), r, p, p) @ w["x_embedder.proj.1.weight"].numpy().T
    mu = h.mean(-1, keepdims=True)
    y = (h - mu) / np.sqrt(((h - mu) ** 2).mean(-1, keepdims=True) + 1e-6) @ w["final_layer.linear.weight"].numpy().T
    np.testing.assert_allclose(out.numpy(), net_oracle.unpatchify_loops(y, p, r, C_out), atol=1e-11)
    assert tout.abs().max().item() < 1e-12


@pytest.mark.parametrize("lora_dim", [0, 8])
def test_network_grads_adjoint_identity_and_weight_differences(net_oracle, lora_dim):
    """Reverse mode: <dout, J tx> = <dx, tx> with J tx from the pinned forward mode; weight gradients against central
    differences of <dout, out> in one entry of a weight of every kind."""
    B, C, C_out, D, H, Kc, p, r, Mk = 1, 2, 2, 16, 2, 12, 2, 1, 4
    T, Hh, W = 2, 4, 4
    w = make_network_weights(C=C, C_out=C_out, D=D, H=H, Kc=Kc, p=p, r=r, n_blocks=2, lora_dim=lora_dim, mask=True, extra=True, seed=21)
    i = make_inputs(B, C, T, Hh, W, T, Mk, Kc, 22)
    halfang = np.random.default_rng(23).standard_normal((T * 2 * 2, D // H // 2))
    angles = np.concatenate([halfang, halfang], -1)
    kw = dict(num_heads=H, patch_spatial=p, patch_temporal=r, rope_angles=angles, padding_mask=i["pm"], dtype=torch.float64)
    dout = torch.randn(B, C_out, T, Hh, W, generator=torch.Generator().manual_seed(24), dtype=torch.float64)
    dx, dw = net_oracle.network_grads_torch(w, i["x"], i["ts"], i["ctx"], dout, **kw)
    _, tout = net_oracle.network_torch(w, i["x"], i["ts"], i["ctx"], tx=i["tx"], **kw)
    lhs, rhs = float((dout * tout).sum()), float((dx * i["tx"]).sum())
    assert abs(lhs - rhs) <= 1e-9 * max(1.0, abs(lhs)), (lhs, rhs)
    assert not any(k.startswith("pos_embedder.") for k in dw)
    eps = 1e-6
    names = ["x_embedder.proj.1.weight", "t_embedder.1.linear_1.weight", "t_embedder.1.linear_2.weight", "t_embedding_norm.weight",
             "blocks.0.self_attn.q_proj.weight", "blocks.1.cross_attn.k_norm.weight", "blocks.1.mlp.layer2.weight",
             "blocks.0.adaln_modulation_mlp.1.weight", "final_layer.adaln_modulation.1.weight", "final_layer.linear.weight",
             "extra_pos_embedder.pos_emb_h"]
    for n, name in enumerate(names):
        idx = tuple(int(v) % s for v, s in zip((3 + n, 5 + 2 * n), w[name].shape))
        vals = []
        for sign in (1, -1):
            w2 = dict(w)
            w2[name] = w[name].clone()
            w2[name][idx] += sign * eps
            out, _ = net_oracle.network_torch(w2, i["x"], i["ts"], i["ctx"], **kw)
            vals.append(float((dout * out).sum()))
        fd = (vals[0] - vals[1]) / (2 * eps)
        got = float(dw[name][idx])
        assert abs(fd - got) <= 1e-5 * max(1.0, abs(fd)), (name, idx, fd, got)
