"""CPU oracle for the DiT network around the blocks (patch embedding, sinusoidal time embedding and its MLP, RMSNorm of
the embedding, optional per-block learned position term, blocks, final LayerNorm + modulation + projection, unpatchify)
and its forward-mode tangent along (x, timesteps).

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module; only ``tests/``,
``__graft_entry__.smoke()`` and ``bench.py`` may use it, as the checker.

What it restates: ``MiniTrainDIT.forward`` of cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:1572-1658 with
``prepare_embedded_sequence`` :1513-1560 (padding-mask channel :1541-1547, patchify ``b c (t r) (h m) (w n) -> b t h w
(c r m n)`` :862-867), ``Timesteps`` :727-743 (``cat([cos, sin])``, frequencies ``10000 ** (-i / half)``),
``TimestepEmbedding`` :777-790 (with adaLN-LoRA the sinusoidal features themselves are the embedding and the MLP output
is the LoRA term), ``t_embedding_norm`` :1417, ``LearnablePosEmbAxis.generate_embeddings`` :698-715, ``FinalLayer.forward``
:960-989 (LoRA term ``[:, :, :2 D]``), ``unpatchify`` ``B T H W (p1 p2 t C) -> B C (T t) (H p1) (W p2)`` :1562-1570.
Written as one pure torch function so that ``torch.func.jvp`` gives the tangent; the blocks are
``dit_block_oracle.make_block_forward``.

Parity status: pinned in tests/test_oracle_dit_network.py -- the patchify / unpatchify index maps by brute-force loops,
the time embedding against explicit numpy fp64, central finite differences (fp64) for the tangent, and the
initialisation property (final modulation zero, LoRA zero => output is ``linear(layer_norm(x))``).
``network_grads_torch`` (torch autograd of the same function): the adjoint identity against the pinned tangent and
finite differences in weights of every kind.
``t_embedding_norm`` is Transformer Engine's RMSNorm in the reference (absent here): PARITY UNPINNED against that
library itself; it is restated as ``x * rsqrt(mean(x^2) + eps) * weight``.
"""
from __future__ import annotations

import importlib.util
import math
import os
from typing import Dict

_block_oracle = None


def _block():
    global _block_oracle
    if _block_oracle is None:
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dit_block_oracle.py")
        spec = importlib.util.spec_from_file_location("_dit_block_oracle_for_network", path)
        _block_oracle = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(_block_oracle)
    return _block_oracle


def patchify_loops(x, r: int, m: int, n: int):
    """``b c (t r) (h m) (w n) -> b t h w (c r m n)`` by explicit index arithmetic (numpy; small inputs)."""
    import numpy as np

    x = np.asarray(x)
    B, C, T, H, W = x.shape
    out = np.zeros((B, T // r, H // m, W // n, C * r * m * n), x.dtype)
    for c in range(C):
        for ir in range(r):
            for im in range(m):
                for in_ in range(n):
                    ch = ((c * r + ir) * m + im) * n + in_
                    out[..., ch] = x[:, c, ir::r, im::m, in_::n]
    return out


def unpatchify_loops(y, p: int, t: int, C: int):
    """``B T H W (p1 p2 t C) -> B C (T t) (H p1) (W p2)`` by explicit index arithmetic (numpy; small inputs)."""
    import numpy as np

    y = np.asarray(y)
    B, T, H, W, _ = y.shape
    out = np.zeros((B, C, T * t, H * p, W * p), y.dtype)
    for p1 in range(p):
        for p2 in range(p):
            for it in range(t):
                for c in range(C):
                    ch = ((p1 * p + p2) * t + it) * C + c
                    out[:, c, it::t, p1::p, p2::p] = y[..., ch]
    return out


def _make_network_forward(w, B, C, T, H, W, *, num_heads, p, r, a, ctx, pm, img, dt):
    """The network as a pure function ``fwd(x [B,C,T,H,W], ts [B,T']) -> [B,C_out,T,H,W]`` of CPU torch tensors of one
    dtype (w: state dict, possibly of tensors that require grad)."""
    import torch
    import torch.nn.functional as F

    D = w["x_embedder.proj.1.weight"].shape[0]
    use_lora = "final_layer.adaln_modulation.2.weight" in w
    n_blocks = 1 + max(int(k.split(".")[1]) for k in w if k.startswith("blocks."))
    C_out = w["final_layer.linear.weight"].shape[0] // (p * p * r)

    if "crossattn_proj.0.weight" in w:
        ctx = F.gelu(F.linear(ctx, w["crossattn_proj.0.weight"], w["crossattn_proj.0.bias"]))
    if img is not None:
        img = F.gelu(F.linear(img, w["img_context_proj.0.weight"], w["img_context_proj.0.bias"]))
    extra = None
    if "extra_pos_embedder.pos_emb_h" in w:
        Tp, Hp, Wp = T // r, H // p, W // p
        e = (w["extra_pos_embedder.pos_emb_t"][:Tp, None, None] + w["extra_pos_embedder.pos_emb_h"][None, :Hp, None]
             + w["extra_pos_embedder.pos_emb_w"][None, None, :Wp])
        norm = e.pow(2).sum(-1, keepdim=True).sqrt()
        extra = (e / (1e-6 + norm / math.sqrt(D)))[None].expand(B, -1, -1, -1, -1)
    mask_channel = None
    if w["x_embedder.proj.1.weight"].shape[1] == (C + 1) * p * p * r:
        mask_channel = F.interpolate(pm, size=[H, W], mode="nearest")[:, :, None].expand(B, 1, T, H, W)
    blocks = [_block().make_block_forward({k[len(f"blocks.{i}."):]: v for k, v in w.items() if k.startswith(f"blocks.{i}.")},
                                          num_heads, a, ctx, img) for i in range(n_blocks)]
    half = D // 2
    freqs = torch.exp(-math.log(10000.0) * torch.arange(half, dtype=dt) / half)

    def fwd(x_, ts_):
        if mask_channel is not None:
            x_ = torch.cat([x_, mask_channel], dim=1)
        c = x_.shape[1]
        h = x_.reshape(B, c, T // r, r, H // p, p, W // p, p).permute(0, 2, 4, 6, 1, 3, 5, 7).reshape(B, T // r, H // p, W // p, c * r * p * p)
        h = F.linear(h, w["x_embedder.proj.1.weight"])
        ang = ts_[..., None] * freqs
        sample = torch.cat([torch.cos(ang), torch.sin(ang)], dim=-1)
        mlp = F.linear(F.silu(F.linear(sample, w["t_embedder.1.linear_1.weight"], w.get("t_embedder.1.linear_1.bias"))),
                       w["t_embedder.1.linear_2.weight"])
        emb, lora = (sample, mlp) if use_lora else (mlp, torch.zeros((), dtype=dt))
        emb = emb * torch.rsqrt(emb.pow(2).mean(-1, keepdim=True) + 1e-6) * w["t_embedding_norm.weight"]
        for blk in blocks:
            h = blk(h if extra is None else h + extra, emb, lora)
        m = F.linear(F.silu(emb), w["final_layer.adaln_modulation.1.weight"])
        if use_lora:
            m = F.linear(m, w["final_layer.adaln_modulation.2.weight"]) + lora[:, :, : 2 * D]
        shift, scale = (z[:, :, None, None, :] for z in m.chunk(2, dim=-1))
        y = F.linear(F.layer_norm(h, (D,), eps=1e-6) * (1 + scale) + shift, w["final_layer.linear.weight"])
        y = y.reshape(B, T // r, H // p, W // p, p, p, r, C_out)
        return y.permute(0, 7, 1, 6, 2, 4, 3, 5).reshape(B, C_out, T, H, W)

    return fwd


def network_torch(weights: Dict[str, "torch.Tensor"], x, timesteps, crossattn_emb, *, num_heads: int, patch_spatial: int,
                  patch_temporal: int, rope_angles=None, padding_mask=None, img_context_emb=None, tx=None, ttimesteps=None,
                  dtype=None):
    """weights: the network's state dict.  x: [B, C, T, H, W]; timesteps: [B, T'] (T' = 1 or T / patch_temporal);
    crossattn_emb: [B, Mk, Kc]; rope_angles: [T'*H'*W', head_dim]; padding_mask: [B, 1, h, w] (required iff the patch
    embedding has one more input channel than x).  Returns (out [B, C_out, T, H, W], tout or None)."""
    import torch

    dt = dtype or torch.float32
    f = lambda t: None if t is None else torch.as_tensor(t).detach().to("cpu", dt)
    w = {k: f(v) for k, v in weights.items() if torch.is_floating_point(v)}
    x, ts, ctx, a, pm, img, tx, tts = (f(t) for t in (x, timesteps, crossattn_emb, rope_angles, padding_mask, img_context_emb, tx, ttimesteps))
    B, C, T, H, W = x.shape
    fwd = _make_network_forward(w, B, C, T, H, W, num_heads=num_heads, p=patch_spatial, r=patch_temporal, a=a, ctx=ctx, pm=pm, img=img, dt=dt)
    if ts.ndim == 1:
        ts = ts[:, None]
    if tx is None:
        return fwd(x, ts), None
    tts = torch.zeros_like(ts) if tts is None else tts.reshape(ts.shape)
    return torch.func.jvp(fwd, (x, ts), (tx, tts))


def network_grads_torch(weights: Dict[str, "torch.Tensor"], x, timesteps, crossattn_emb, dout, *, num_heads: int, patch_spatial: int,
                        patch_temporal: int, rope_angles=None, padding_mask=None, dtype=None):
    """Reverse mode of the same function by torch autograd: (dx, {weight name: gradient}) for the cotangent ``dout`` of the
    output.  Weights that the output does not depend on (position tables) are left out."""
    import torch

    dt = dtype or torch.float32
    f = lambda t: None if t is None else torch.as_tensor(t).detach().to("cpu", dt)
    w = {k: f(v).requires_grad_(True) for k, v in weights.items() if torch.is_floating_point(v) and not k.startswith("pos_embedder.")}
    x, ts, ctx, a, pm, dout = (f(t) for t in (x, timesteps, crossattn_emb, rope_angles, padding_mask, dout))
    x.requires_grad_(True)
    B, C, T, H, W = x.shape
    fwd = _make_network_forward(w, B, C, T, H, W, num_heads=num_heads, p=patch_spatial, r=patch_temporal, a=a, ctx=ctx, pm=pm, img=None, dt=dt)
    out = fwd(x, ts if ts.ndim == 2 else ts[:, None])
    names = list(w)
    grads = torch.autograd.grad(out, [x] + [w[k] for k in names], grad_outputs=dout, allow_unused=True)
    return grads[0], {k: g for k, g in zip(names, grads[1:]) if g is not None}
