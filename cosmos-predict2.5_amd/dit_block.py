"""The DiT transformer ``Block`` (self-attention, cross-attention and MLP, each behind a LayerNorm with adaLN
modulation and a gated residual) on the HIP attention path, with a forward that also carries a tangent.

Reference: ``Block`` (cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:993-1242) and ``GPT2FeedForward``
(:222-249) -- same constructor arguments, sub-module and parameter names (``self_attn.*``, ``cross_attn.*``,
``mlp.layer1/2.weight``, ``adaln_modulation_{self_attn,cross_attn,mlp}.{1,2}.weight``: a reference state dict of the
block loads as is), ``init_weights``, ``forward(x_B_T_H_W_D, emb_B_T_D, crossattn_emb, rope_emb_L_1_1_D,
adaln_lora_B_T_3D, extra_per_block_pos_emb)``.

``forward_jvp`` pushes a tangent of ``(x, emb, adaln_lora)`` through the block: what a consistency-distillation step
needs when it differentiates the network along (x_t, t).  The reference ships the attention JVP kernel but no caller
that does this, so the rules are written out here: LayerNorm + modulation, GELU and the gated residuals each in one
fused HIP pass (fp32 arithmetic on 16-bit tensors), the tiny modulation MLP by torch forward AD, linear layers on
primal and tangent stacked in one GEMM (the fused passes write both into one buffer, so nothing is copied to stack
them), attention through ``Attention.forward_jvp``.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import nn

from . import ops
from .dit_attention import Attention, I2VCrossAttention


class _LnModulateFn(torch.autograd.Function):
    """``LayerNorm(x) * (1 + scale) + shift`` as the fused pass, differentiable: the backward pass recomputes the
    expression in fp32 with tensor-library ops and takes their gradients (x ``[B, T, H, W, D]``, shift / scale
    ``[B, T, 1, 1, D]``)."""

    @staticmethod
    def forward(ctx, x, shift, scale, eps):
        D = x.shape[-1]
        y, _ = ops.ln_modulate(x, shift.reshape(-1, D), scale.reshape(-1, D), eps=eps)
        ctx.save_for_backward(x, shift, scale)
        ctx.eps = eps
        return y

    @staticmethod
    def backward(ctx, dy):
        x, shift, scale = ctx.saved_tensors
        with torch.enable_grad():
            xf, sh, sc = (t.detach().float().requires_grad_(True) for t in (x, shift, scale))
            y = F.layer_norm(xf, (x.shape[-1],), eps=ctx.eps) * (1 + sc) + sh
        dx, dsh, dsc = torch.autograd.grad(y, (xf, sh, sc), dy.float())
        return dx.to(x.dtype), dsh.to(shift.dtype), dsc.to(scale.dtype), None


class _GatedResidualFn(torch.autograd.Function):
    """``x + gate * res`` as the fused pass, differentiable (gate ``[B, T, 1, 1, D]``)."""

    @staticmethod
    def forward(ctx, x, res, gate):
        out, _ = ops.gated_residual(x, res, gate.reshape(-1, x.shape[-1]))
        ctx.save_for_backward(res, gate)
        return out

    @staticmethod
    def backward(ctx, dy):
        res, gate = ctx.saved_tensors
        dgate = (dy.float() * res.float()).sum(dim=(2, 3), keepdim=True).to(gate.dtype)
        return dy, dy * gate, dgate


class _GeluFn(torch.autograd.Function):
    """Exact GELU as the fused pass, differentiable."""

    @staticmethod
    def forward(ctx, h):
        ctx.save_for_backward(h)
        return ops.gelu(h)[0]

    @staticmethod
    def backward(ctx, dy):
        (h,) = ctx.saved_tensors
        return torch.ops.aten.gelu_backward(dy, h, approximate="none")


class GPT2FeedForward(nn.Module):
    def __init__(self, d_model: int, d_ff: int):
        super().__init__()
        self.activation = nn.GELU()
        self.layer1 = nn.Linear(d_model, d_ff, bias=False)
        self.layer2 = nn.Linear(d_ff, d_model, bias=False)
        self._layer_id = None
        self._dim = d_model
        self._hidden_dim = d_ff
        self.init_weights()

    def init_weights(self) -> None:
        """minimal_v4_dit.py:234-242: truncated normal, std 1/sqrt(fan_in), the second layer scaled down with depth."""
        std = 1.0 / math.sqrt(self._dim)
        torch.nn.init.trunc_normal_(self.layer1.weight, std=std, a=-3 * std, b=3 * std)
        std = 1.0 / math.sqrt(self._hidden_dim)
        if self._layer_id is not None:
            std = std / math.sqrt(2 * (self._layer_id + 1))
        torch.nn.init.trunc_normal_(self.layer2.weight, std=std, a=-3 * std, b=3 * std)

    def forward(self, x: torch.Tensor):
        h = self.layer1(x)
        if h.is_cuda and h.numel() % 8 == 0 and h.dtype in (torch.bfloat16, torch.float16):
            if torch.is_grad_enabled() and h.requires_grad:
                return self.layer2(_GeluFn.apply(h))
            return self.layer2(ops.gelu(h, inplace=True)[0])      # inference: one fused pass, in place
        return self.layer2(self.activation(h))

    @torch.no_grad()
    def forward_jvp(self, x: torch.Tensor, tx: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        b = x.shape[0]
        both = ops.as_stacked(x, tx)
        h = self.layer1(both if both is not None else torch.cat([x, tx], dim=0))
        ops.gelu(h[:b], h[b:], inplace=True)       # a = gelu(h), ta = th gelu'(h), in place on the stacked buffer
        y = self.layer2(h)
        return y[:b], y[b:]


class Block(nn.Module):
    def __init__(
        self,
        x_dim: int,
        context_dim: int,
        num_heads: int,
        mlp_ratio: float = 4.0,
        use_adaln_lora: bool = False,
        adaln_lora_dim: int = 256,
        backend: str = "hip",
        image_context_dim: Optional[int] = None,
        use_wan_fp32_strategy: bool = False,
    ):
        super().__init__()
        self.x_dim = x_dim
        fp32 = dict(use_wan_fp32_strategy=use_wan_fp32_strategy)
        self.layer_norm_self_attn = nn.LayerNorm(x_dim, elementwise_affine=False, eps=1e-6)
        self.self_attn = Attention(x_dim, None, num_heads, x_dim // num_heads, qkv_format="bshd", backend=backend, **fp32)
        self.layer_norm_cross_attn = nn.LayerNorm(x_dim, elementwise_affine=False, eps=1e-6)
        if image_context_dim is None:
            self.cross_attn = Attention(x_dim, context_dim, num_heads, x_dim // num_heads, qkv_format="bshd", backend=backend, **fp32)
        else:   # crossattn_emb is then the pair (text context, image context)
            self.cross_attn = I2VCrossAttention(x_dim, context_dim, num_heads, x_dim // num_heads,
                                                img_latent_dim=image_context_dim, qkv_format="bshd", backend=backend, **fp32)
        self.layer_norm_mlp = nn.LayerNorm(x_dim, elementwise_affine=False, eps=1e-6)
        self.mlp = GPT2FeedForward(x_dim, int(x_dim * mlp_ratio))

        self.use_adaln_lora = use_adaln_lora

        def modulation():
            if use_adaln_lora:
                return nn.Sequential(nn.SiLU(), nn.Linear(x_dim, adaln_lora_dim, bias=False),
                                     nn.Linear(adaln_lora_dim, 3 * x_dim, bias=False))
            return nn.Sequential(nn.SiLU(), nn.Linear(x_dim, 3 * x_dim, bias=False))

        self.adaln_modulation_self_attn = modulation()
        self.adaln_modulation_cross_attn = modulation()
        self.adaln_modulation_mlp = modulation()
        self.cp_size = None
        self.use_wan_fp32_strategy = use_wan_fp32_strategy

    def set_context_parallel_group(self, process_group, ranks, stream):
        self.cp_size = None if ranks is None else len(ranks)
        self.self_attn.set_context_parallel_group(process_group=process_group, ranks=ranks, stream=stream)

    def reset_parameters(self) -> None:
        """minimal_v4_dit.py:1095-1111: the last modulation layer starts at zero (the block starts as the identity)."""
        mods = (self.adaln_modulation_self_attn, self.adaln_modulation_cross_attn, self.adaln_modulation_mlp)
        if self.use_adaln_lora:
            std = 1.0 / math.sqrt(self.x_dim)
            for m in mods:
                torch.nn.init.trunc_normal_(m[1].weight, std=std, a=-3 * std, b=3 * std)
                torch.nn.init.zeros_(m[2].weight)
        else:
            for m in mods:
                torch.nn.init.zeros_(m[1].weight)

    def init_weights(self) -> None:
        self.reset_parameters()
        self.self_attn.init_weights()
        self.cross_attn.init_weights()
        self.mlp.init_weights()

    # ------------------------------------------------------------------ pieces
    def _modulation(self, mod: nn.Sequential, emb_B_T_D, adaln_lora_B_T_3D, like):
        """(shift, scale, gate), each ``[B, T, 1, 1, D]`` in the type of x (minimal_v4_dit.py:1131-1162).  With
        ``use_wan_fp32_strategy`` the modulation MLP runs in fp32 (an fp32 autocast region, as in the reference) on the
        fp32 time embedding and is rounded once, to the type of x."""
        with self._fp32_region(emb_B_T_D):
            m = mod(emb_B_T_D)
            if self.use_adaln_lora:
                m = m + adaln_lora_B_T_3D
        return tuple(c[:, :, None, None, :].type_as(like) for c in m.chunk(3, dim=-1))

    def _modulation_jvp(self, mod: nn.Sequential, emb, temb, lora, tlora, like):
        """Modulation and its tangent; the tensors are ``[B, T, 3 D]``, tiny next to x: forward AD does it."""
        f = (lambda e, l: mod(e) + l) if self.use_adaln_lora else (lambda e, l: mod(e))
        if lora is None:
            lora = emb.new_zeros(())
        temb = torch.zeros_like(emb) if temb is None else temb
        tlora = torch.zeros_like(lora) if tlora is None else tlora
        with self._fp32_region(emb):
            m, tm = torch.func.jvp(f, (emb, lora), (temb, tlora))
        cut = lambda z: tuple(c[:, :, None, None, :].type_as(like) for c in z.chunk(3, dim=-1))
        return cut(m), cut(tm)

    def _fp32_region(self, t: torch.Tensor):
        return torch.autocast(t.device.type, enabled=self.use_wan_fp32_strategy, dtype=torch.float32)

    @staticmethod
    def _modulate_jvp(norm_layer, x, tx, mod, tmod):
        """LayerNorm + modulation of x and its tangent (one fused pass), written into the two halves of one buffer so
        that the projections that follow map both in one GEMM without a copy."""
        (shift, scale, _), (tshift, tscale, _) = mod, tmod
        y, ty = ops.stacked_pair(x.shape, x.dtype, x.device)
        flat = lambda m: m.reshape(-1, m.shape[-1])
        ops.ln_modulate(x, flat(shift), flat(scale), tx, flat(tshift), flat(tscale), eps=norm_layer.eps, out=y, tout=ty)
        return y, ty

    @staticmethod
    def _gated_residual_jvp(x, tx, res, tres, mod, tmod):
        flat = lambda m: m.reshape(-1, m.shape[-1])
        return ops.gated_residual(x, res, flat(mod[2]), tx, tres, flat(tmod[2]))

    # ------------------------------------------------------------------ the reference's surface
    def forward(
        self,
        x_B_T_H_W_D: torch.Tensor,
        emb_B_T_D: torch.Tensor,
        crossattn_emb: torch.Tensor,
        rope_emb_L_1_1_D: Optional[torch.Tensor] = None,
        adaln_lora_B_T_3D: Optional[torch.Tensor] = None,
        extra_per_block_pos_emb: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        x = x_B_T_H_W_D
        if extra_per_block_pos_emb is not None:
            x = x + extra_per_block_pos_emb
        if not torch.is_grad_enabled() and x.is_cuda:
            return self._forward_fused(x, emb_B_T_D, crossattn_emb, rope_emb_L_1_1_D, adaln_lora_B_T_3D)
        return self._forward_autograd(x, emb_B_T_D, crossattn_emb, rope_emb_L_1_1_D, adaln_lora_B_T_3D)

    def _forward_autograd(self, x, emb, crossattn_emb, rope, lora):
        """The differentiable path: the same kernels as the inference path (so both give the same bits), each behind an
        autograd rule -- attention and RMSNorm + RoPE through their HIP backward kernels, the elementwise passes through
        fp32 tensor-library arithmetic."""
        B, T, H, W, D = x.shape
        for name, norm, sub in (("self_attn", self.layer_norm_self_attn, self.self_attn),
                                ("cross_attn", self.layer_norm_cross_attn, self.cross_attn),
                                ("mlp", self.layer_norm_mlp, self.mlp)):
            shift, scale, gate = self._modulation(getattr(self, "adaln_modulation_" + name), emb, lora, x)
            n = _LnModulateFn.apply(x, shift, scale, norm.eps)
            if name == "mlp":
                r = sub(n)
            else:
                r = sub(n.reshape(B, T * H * W, D), None if name == "self_attn" else crossattn_emb, rope_emb=rope)
            x = _GatedResidualFn.apply(x, r.reshape(x.shape), gate)
        return x

    def _forward_fused(self, x, emb, crossattn_emb, rope, lora):
        """Inference (no autograd): the same arithmetic with LayerNorm + modulation, the gated residuals and GELU each as
        one fused HIP pass instead of a chain of tensor-library ops."""
        B, T, H, W, D = x.shape
        flat2 = lambda m: m.reshape(-1, D)
        for name, norm, sub in (("self_attn", self.layer_norm_self_attn, self.self_attn),
                                ("cross_attn", self.layer_norm_cross_attn, self.cross_attn),
                                ("mlp", self.layer_norm_mlp, self.mlp)):
            shift, scale, gate = self._modulation(getattr(self, "adaln_modulation_" + name), emb, lora, x)
            n, _ = ops.ln_modulate(x, flat2(shift), flat2(scale), eps=norm.eps)
            if name == "mlp":
                r = sub(n)
            else:
                r = sub(n.reshape(B, T * H * W, D), None if name == "self_attn" else crossattn_emb, rope_emb=rope)
            x, _ = ops.gated_residual(x, r.reshape(x.shape), flat2(gate))
        return x

    # ------------------------------------------------------------------ forward mode
    @torch.no_grad()
    def forward_jvp(
        self,
        x_B_T_H_W_D: torch.Tensor,
        tx_B_T_H_W_D: torch.Tensor,
        emb_B_T_D: torch.Tensor,
        temb_B_T_D: Optional[torch.Tensor],
        crossattn_emb: torch.Tensor,
        rope_emb_L_1_1_D: Optional[torch.Tensor] = None,
        adaln_lora_B_T_3D: Optional[torch.Tensor] = None,
        tadaln_lora_B_T_3D: Optional[torch.Tensor] = None,
        extra_per_block_pos_emb: Optional[torch.Tensor] = None,
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        """``(out, tout)``: the block's output and its derivative along ``(tx, temb, tadaln_lora)``; the text context
        and the positional terms do not move."""
        x, tx = x_B_T_H_W_D, tx_B_T_H_W_D
        assert tx.shape == x.shape
        if extra_per_block_pos_emb is not None:
            x = x + extra_per_block_pos_emb
        B, T, H, W, D = x.shape
        flat = lambda z: z.reshape(B, T * H * W, D)
        vid = lambda z: z.reshape(B, T, H, W, D)
        args = (emb_B_T_D, temb_B_T_D, adaln_lora_B_T_3D, tadaln_lora_B_T_3D, x)

        mod, tmod = self._modulation_jvp(self.adaln_modulation_self_attn, *args)
        n, tn = self._modulate_jvp(self.layer_norm_self_attn, x, tx, mod, tmod)
        r, tr = self.self_attn.forward_jvp(flat(n), flat(tn), rope_emb=rope_emb_L_1_1_D)
        x, tx = self._gated_residual_jvp(x, tx, vid(r), vid(tr), mod, tmod)

        mod, tmod = self._modulation_jvp(self.adaln_modulation_cross_attn, *args)
        n, tn = self._modulate_jvp(self.layer_norm_cross_attn, x, tx, mod, tmod)
        r, tr = self.cross_attn.forward_jvp(flat(n), flat(tn), crossattn_emb, None, rope_emb=rope_emb_L_1_1_D)
        x, tx = self._gated_residual_jvp(x, tx, vid(r), vid(tr), mod, tmod)

        mod, tmod = self._modulation_jvp(self.adaln_modulation_mlp, *args)
        n, tn = self._modulate_jvp(self.layer_norm_mlp, x, tx, mod, tmod)
        r, tr = self.mlp.forward_jvp(n, tn)
        x, tx = self._gated_residual_jvp(x, tx, r, tr, mod, tmod)
        return x, tx
