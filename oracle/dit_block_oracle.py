"""CPU oracle for the DiT transformer block (adaLN-modulated self-attention, cross-attention and MLP with gated
residuals) and its forward-mode tangent.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module; only ``tests/``,
``__graft_entry__.smoke()`` and ``bench.py`` may use it, as the checker.

What it restates: ``Block.forward`` of cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:1119-1242 (modulation
:1131-1162 with chunk order shift, scale, gate; ``norm(x) * (1 + scale) + shift`` :1166-1167; gated residuals :1199,
:1231, :1241), ``GPT2FeedForward.forward`` :244-249 (exact GELU), ``Attention.forward`` with the torch backend
(see dit_attention_oracle.py), written as one pure torch function so that ``torch.func.jvp`` gives the tangent.
LayerNorm, GELU, SiLU, linear layers and SDPA are the library routines themselves.

``ln_modulate_torch``, ``gated_residual_torch``, ``gelu_torch``: the three elementwise steps on their own (library
``layer_norm`` / ``gelu`` under ``torch.func.jvp``), the checkers of the fused kernels.

Parity status: pinned in tests/test_oracle_dit_block.py -- a step-by-step fp64 numpy recomputation with explicit
statistics (and the separately pinned attention-module oracle for the two attention calls), central finite
differences for the tangent, and the reference's initialisation property (last modulation layer zero => the block is
the identity).  RMSNorm / RoPE inside the attention modules: see norm_rope_oracle.py (PARITY UNPINNED against
Transformer Engine itself).
"""
from __future__ import annotations

from typing import Dict, Optional


def make_block_forward(w, num_heads: int, rope_angles, ctx, img_ctx=None):
    """The block as a pure function ``fwd(x [B,T,H,W,D], emb [B,T,D], adaln_lora [B,T,3D] or 0-d) -> [B,T,H,W,D]`` of
    torch tensors that already sit on the CPU in one dtype (w: state dict; rope_angles: [T*H*W, head_dim] or None;
    ctx: text context; img_ctx: image context or None)."""
    import torch
    import torch.nn.functional as F
    from torch.nn.attention import SDPBackend, sdpa_kernel

    use_lora = "adaln_modulation_mlp.2.weight" in w
    D = w["mlp.layer2.weight"].shape[0]
    hd = D // num_heads
    a = None if rope_angles is None else rope_angles.reshape(1, -1, 1, hd)

    def modulation(name, e, l):
        m = F.linear(F.silu(e), w[f"adaln_modulation_{name}.1.weight"])
        if use_lora:
            m = F.linear(m, w[f"adaln_modulation_{name}.2.weight"]) + l
        return [c[:, :, None, None, :] for c in m.chunk(3, dim=-1)]     # shift, scale, gate

    def norm_rope(t, g, rope):
        n = F.rms_norm(t, (hd,), weight=g, eps=1e-6)
        if rope is None:
            return n
        return n * torch.cos(rope) + torch.cat([-n[..., hd // 2:], n[..., : hd // 2]], dim=-1) * torch.sin(rope)

    def attention(prefix, xq, c, rope, c_img=None):
        heads = lambda t: t.reshape(t.shape[0], -1, num_heads, hd)
        sdpa = lambda q_, k_, v_: F.scaled_dot_product_attention(q_.transpose(1, 2), k_.transpose(1, 2), v_.transpose(1, 2)).transpose(1, 2)
        q = norm_rope(heads(F.linear(xq, w[prefix + "q_proj.weight"])), w[prefix + "q_norm.weight"], rope)
        k = norm_rope(heads(F.linear(c, w[prefix + "k_proj.weight"])), w[prefix + "k_norm.weight"], rope)
        v = heads(F.linear(c, w[prefix + "v_proj.weight"]))
        with sdpa_kernel([SDPBackend.MATH]):
            o = sdpa(q, k, v)
            if c_img is not None:
                k_img = norm_rope(heads(F.linear(c_img, w[prefix + "k_img.weight"])), w[prefix + "k_img_norm.weight"], None)
                o = o + sdpa(q, k_img, heads(F.linear(c_img, w[prefix + "v_img.weight"])))
        return F.linear(o.flatten(-2), w[prefix + "output_proj.weight"])

    def fwd(x_, e_, l_):
        B, T, H, W, _ = x_.shape
        ln = lambda t: F.layer_norm(t, (D,), eps=1e-6)
        shift, scale, gate = modulation("self_attn", e_, l_)
        n = (ln(x_) * (1 + scale) + shift).reshape(B, T * H * W, D)
        x_ = x_ + gate * attention("self_attn.", n, n, a).reshape(B, T, H, W, D)
        shift, scale, gate = modulation("cross_attn", e_, l_)
        n = (ln(x_) * (1 + scale) + shift).reshape(B, T * H * W, D)
        x_ = attention("cross_attn.", n, ctx, None, img_ctx).reshape(B, T, H, W, D) * gate + x_
        shift, scale, gate = modulation("mlp", e_, l_)
        n = ln(x_) * (1 + scale) + shift
        return x_ + gate * F.linear(F.gelu(F.linear(n, w["mlp.layer1.weight"])), w["mlp.layer2.weight"])

    return fwd


def block_torch(weights: Dict[str, "torch.Tensor"], x, emb, crossattn_emb, rope_angles=None, num_heads: int = 8,
                adaln_lora=None, tx=None, temb=None, tadaln_lora=None, dtype=None, keep_graph_input=None):
    """weights: the block's state dict.  x: [B, T, H, W, D]; emb: [B, T, D]; crossattn_emb: [B, Mk, Kc], or the pair
    (text context, image context [B, Mi, Ki]) when the state dict holds the image-conditioned cross-attention
    (``cross_attn.k_img.weight`` ...: minimal_v4_dit.py:451-493, the two attention results are summed before the output
    projection);
    rope_angles: [T*H*W, D/num_heads] or None; adaln_lora: [B, T, 3 D] (required iff the state dict holds the
    LoRA form of the modulation).  Returns (out, tout); tout is None without tx."""
    import torch

    dt = dtype or torch.float32
    f = lambda t: None if t is None else torch.as_tensor(t).detach().to("cpu", dt)
    w = {k: f(v) for k, v in weights.items()}
    img_ctx = None
    if isinstance(crossattn_emb, (tuple, list)):
        crossattn_emb, img_ctx = crossattn_emb
        img_ctx = f(img_ctx)
    x, emb, ctx, lora, tx, temb, tlora = (f(t) for t in (x, emb, crossattn_emb, adaln_lora, tx, temb, tadaln_lora))
    if keep_graph_input is not None:
        x = keep_graph_input.to(dt)
    a = None if rope_angles is None else f(rope_angles)
    fwd = make_block_forward(w, num_heads, a, ctx, img_ctx)

    if lora is None:
        lora = torch.zeros((), dtype=dt)
    if tx is None:
        return fwd(x, emb, lora), None
    temb = torch.zeros_like(emb) if temb is None else temb
    tlora = torch.zeros_like(lora) if tlora is None else tlora
    return torch.func.jvp(fwd, (x, emb, lora), (tx, temb, tlora))


def ln_modulate_torch(x, shift, scale, tx=None, tshift=None, tscale=None, eps: float = 1e-6, rows_per_group: int = 1):
    """fp32: ``layer_norm(x) * (1 + scale) + shift`` over the last dim with [G, D] modulation vectors shared by
    ``rows_per_group`` consecutive rows of the flattened x; tangent along (tx, tshift, tscale) by forward AD."""
    import torch
    import torch.nn.functional as F

    f32 = lambda t: None if t is None else torch.as_tensor(t).detach().float().cpu()
    x, shift, scale, tx, tshift, tscale = (f32(t) for t in (x, shift, scale, tx, tshift, tscale))
    D = x.shape[-1]
    rep = lambda m: m.reshape(-1, D).repeat_interleave(rows_per_group, dim=0).reshape(x.shape)

    def fn(x_, sh, sc):
        return F.layer_norm(x_, (D,), eps=eps) * (1 + rep(sc)) + rep(sh)

    if tx is None:
        return fn(x, shift, scale), None
    z = lambda t, like: torch.zeros_like(like) if t is None else t
    return torch.func.jvp(fn, (x, shift, scale), (tx, z(tshift, shift), z(tscale, scale)))


def gated_residual_torch(x, res, gate, tx=None, tres=None, tgate=None, rows_per_group: int = 1):
    import torch

    f32 = lambda t: None if t is None else torch.as_tensor(t).detach().float().cpu()
    x, res, gate, tx, tres, tgate = (f32(t) for t in (x, res, gate, tx, tres, tgate))
    D = x.shape[-1]
    rep = lambda m: m.reshape(-1, D).repeat_interleave(rows_per_group, dim=0).reshape(x.shape)
    fn = lambda x_, r_, g_: x_ + rep(g_) * r_
    if tx is None:
        return fn(x, res, gate), None
    return torch.func.jvp(fn, (x, res, gate), (tx, tres, torch.zeros_like(gate) if tgate is None else tgate))


def gelu_torch(h, th=None):
    import torch
    import torch.nn.functional as F

    h = torch.as_tensor(h).detach().float().cpu()
    if th is None:
        return F.gelu(h), None
    return torch.func.jvp(F.gelu, (h,), (torch.as_tensor(th).detach().float().cpu(),))
