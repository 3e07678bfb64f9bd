"""The DiT network around the blocks (patch embedding, time embedding, positional tables, final layer, unpatchify) on
the HIP path, with a forward that also carries a tangent along (x, timesteps).

Reference: ``MiniTrainDIT`` (cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:1245-1658) with its pieces
``Timesteps`` (:722-743), ``TimestepEmbedding`` (:746-783), ``PatchEmbed`` (:841-908), ``FinalLayer`` (:911-990),
``LearnablePosEmbAxis`` (:665-715) -- same constructor arguments (those that select code built here), sub-module and
parameter names (``x_embedder.proj.1.weight``, ``t_embedder.1.linear_{1,2}``, ``t_embedding_norm.weight``,
``blocks.N.*``, ``final_layer.linear / adaln_modulation``, ``crossattn_proj.0``, ``img_context_proj.0``,
``extra_pos_embedder.pos_emb_{h,w,t}``: a reference checkpoint of the network loads as is), and
``forward(x_B_C_T_H_W, timesteps_B_T, crossattn_emb, fps, padding_mask, img_context_emb=...)``; and the
video-conditioned subclass ``MinimalV1LVGDiT`` (networks/minimal_v1_lvg_dit.py:24-62: one more input channel for the
condition mask, ``timestep_scale``).

``forward_jvp`` is what a consistency-distillation step needs: the network output and its derivative along a
direction ``(tx, ttimesteps)`` in one pass (conditioning, positions and padding mask do not move).  The blocks carry the
tangent through their fused kernels (dit_block.Block.forward_jvp); the small pieces around them (time embedding on
``[B, T, D]``) go through torch forward AD, the patch embedding and the final projection map primal and tangent
stacked in one GEMM.

``use_wan_fp32_strategy`` (the released rectified-flow configurations set it): the time embedding, every modulation MLP
and the whole final layer run in fp32 (fp32 autocast regions, as in the reference); timesteps must then arrive in fp32 and
the output is fp32.

``sac_config`` (activation checkpointing): every mode other than "none" checkpoints the blocks: a block keeps its inputs
and the results of its attention calls, everything else is recomputed in the backward pass, which is what lets a 720p
training step fit.

Not built (refused in the constructor): sparse attention (``n_dense_blocks``, ``natten_parameters``); context parallelism
needs a second GPU.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import nn

from . import ops
from .attention import record_attention_results, replay_attention_results
from .dit_block import Block
from .rope_position import VideoRopePosition3DEmb


class Timesteps(nn.Module):
    """Sinusoidal features ``cat([cos, sin])`` of the timesteps, frequencies ``10000 ** (-i / half_dim)`` (:722-743)."""

    def __init__(self, num_channels):
        super().__init__()
        self.num_channels = num_channels

    def forward(self, timesteps_B_T):
        assert timesteps_B_T.ndim == 2, f"Expected 2D input, got {timesteps_B_T.ndim}"
        in_dtype = timesteps_B_T.dtype
        half_dim = self.num_channels // 2
        exponent = -math.log(10000) * torch.arange(half_dim, dtype=torch.float32, device=timesteps_B_T.device) / half_dim
        ang = timesteps_B_T.float()[..., None] * torch.exp(exponent)
        return torch.cat([torch.cos(ang), torch.sin(ang)], dim=-1).to(in_dtype)


class TimestepEmbedding(nn.Module):
    def __init__(self, in_features: int, out_features: int, use_adaln_lora: bool = False):
        super().__init__()
        self.in_dim, self.out_dim = in_features, out_features
        self.linear_1 = nn.Linear(in_features, out_features, bias=not use_adaln_lora)
        self.activation = nn.SiLU()
        self.use_adaln_lora = use_adaln_lora
        self.linear_2 = nn.Linear(out_features, 3 * out_features if use_adaln_lora else out_features, bias=False)
        self.init_weights()

    def init_weights(self) -> None:
        std = 1.0 / math.sqrt(self.in_dim)
        torch.nn.init.trunc_normal_(self.linear_1.weight, std=std, a=-3 * std, b=3 * std)
        std = 1.0 / math.sqrt(self.out_dim)
        torch.nn.init.trunc_normal_(self.linear_2.weight, std=std, a=-3 * std, b=3 * std)

    def forward(self, sample: torch.Tensor):
        """(emb_B_T_D, adaln_lora_B_T_3D): with adaLN-LoRA the embedding is the input itself and the MLP output is the
        LoRA term (:777-783)."""
        emb = self.linear_2(self.activation(self.linear_1(sample)))
        if self.use_adaln_lora:
            return sample, emb
        return emb, None


class RMSNormWeight(nn.Module):
    """RMSNorm over the last dim with a weight (``te.pytorch.RMSNorm(model_channels, eps=1e-6)``, :1417), fp32 arithmetic;
    applied to the ``[B, T, D]`` time embedding only."""

    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def reset_parameters(self) -> None:
        nn.init.ones_(self.weight)

    def forward(self, x):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight.float()).to(x.dtype)


class _Patchify(nn.Module):
    """``b c (t r) (h m) (w n) -> b t h w (c r m n)`` (:862-867)."""

    def __init__(self, r: int, m: int, n: int):
        super().__init__()
        self.r, self.m, self.n = r, m, n

    def forward(self, x):
        B, C, T, H, W = x.shape
        r, m, n = self.r, self.m, self.n
        x = x.reshape(B, C, T // r, r, H // m, m, W // n, n)
        return x.permute(0, 2, 4, 6, 1, 3, 5, 7).reshape(B, T // r, H // m, W // n, C * r * m * n)


class PatchEmbed(nn.Module):
    def __init__(self, spatial_patch_size, temporal_patch_size, in_channels=3, out_channels=768):
        super().__init__()
        self.spatial_patch_size = spatial_patch_size
        self.temporal_patch_size = temporal_patch_size
        self.dim = in_channels * spatial_patch_size * spatial_patch_size * temporal_patch_size
        self.proj = nn.Sequential(_Patchify(temporal_patch_size, spatial_patch_size, spatial_patch_size),
                                  nn.Linear(self.dim, out_channels, bias=False))
        self.init_weights()

    def init_weights(self) -> None:
        std = 1.0 / math.sqrt(self.dim)
        torch.nn.init.trunc_normal_(self.proj[1].weight, std=std, a=-3 * std, b=3 * std)

    def forward(self, x):
        assert x.dim() == 5
        _, _, T, H, W = x.shape
        assert H % self.spatial_patch_size == 0 and W % self.spatial_patch_size == 0, (
            f"H,W {(H, W)} should be divisible by spatial_patch_size {self.spatial_patch_size}"
        )
        assert T % self.temporal_patch_size == 0
        return self.proj(x)


class LearnablePosEmbAxis(nn.Module):
    """Learned per-axis absolute position term added in every block (:665-715), normalised to unit RMS-like norm."""

    def __init__(self, *, interpolation: str, model_channels: int, len_h: int, len_w: int, len_t: int, **kwargs):
        del kwargs
        super().__init__()
        assert interpolation in ["crop"], f"Unknown interpolation method {interpolation}"
        self.interpolation = interpolation
        self.model_channels = model_channels
        self.pos_emb_h = nn.Parameter(torch.zeros(len_h, model_channels))
        self.pos_emb_w = nn.Parameter(torch.zeros(len_w, model_channels))
        self.pos_emb_t = nn.Parameter(torch.zeros(len_t, model_channels))
        self.reset_parameters()

    def reset_parameters(self):
        std = 1.0 / math.sqrt(self.model_channels)
        for p in (self.pos_emb_h, self.pos_emb_w, self.pos_emb_t):
            torch.nn.init.trunc_normal_(p, std=std, a=-3 * std, b=3 * std)

    def forward(self, x_B_T_H_W_C, fps=None):
        del fps
        B, T, H, W, _ = x_B_T_H_W_C.shape
        emb = (self.pos_emb_t[:T, None, None, :] + self.pos_emb_h[None, :H, None, :] + self.pos_emb_w[None, None, :W, :])
        emb = emb[None].expand(B, T, H, W, -1)
        norm = torch.linalg.vector_norm(emb, dim=-1, keepdim=True, dtype=torch.float32)
        norm = torch.add(1e-6, norm, alpha=math.sqrt(norm.numel() / emb.numel()))
        return emb / norm.to(emb.dtype)


class FinalLayer(nn.Module):
    def __init__(self, hidden_size, spatial_patch_size, temporal_patch_size, out_channels, use_adaln_lora: bool = False,
                 adaln_lora_dim: int = 256, use_wan_fp32_strategy: bool = False):
        super().__init__()
        self.use_wan_fp32_strategy = use_wan_fp32_strategy
        self.layer_norm = nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6)
        self.linear = nn.Linear(hidden_size, spatial_patch_size * spatial_patch_size * temporal_patch_size * out_channels, bias=False)
        self.hidden_size = hidden_size
        self.n_adaln_chunks = 2
        self.use_adaln_lora = use_adaln_lora
        self.adaln_lora_dim = adaln_lora_dim
        if use_adaln_lora:
            self.adaln_modulation = nn.Sequential(nn.SiLU(), nn.Linear(hidden_size, adaln_lora_dim, bias=False),
                                                  nn.Linear(adaln_lora_dim, 2 * hidden_size, bias=False))
        else:
            self.adaln_modulation = nn.Sequential(nn.SiLU(), nn.Linear(hidden_size, 2 * hidden_size, bias=False))
        self.init_weights()

    def init_weights(self) -> None:
        std = 1.0 / math.sqrt(self.hidden_size)
        torch.nn.init.trunc_normal_(self.linear.weight, std=std, a=-3 * std, b=3 * std)
        if self.use_adaln_lora:
            torch.nn.init.trunc_normal_(self.adaln_modulation[1].weight, std=std, a=-3 * std, b=3 * std)
            torch.nn.init.zeros_(self.adaln_modulation[2].weight)
        else:
            torch.nn.init.zeros_(self.adaln_modulation[1].weight)

    def _modulation(self, emb_B_T_D, adaln_lora_B_T_3D):
        m = self.adaln_modulation(emb_B_T_D)
        if self.use_adaln_lora:
            assert adaln_lora_B_T_3D is not None
            m = m + adaln_lora_B_T_3D[:, :, : 2 * self.hidden_size]     # (:969-972)
        return m

    def _forward_fp32(self, x_B_T_H_W_D, emb_B_T_D, adaln_lora_B_T_3D):
        """use_wan_fp32_strategy (:967-988): modulation, LayerNorm, modulate and the projection all in fp32 (the autocast
        region lifts the LayerNorm input and the linear layers to fp32); fp32 output."""
        assert emb_B_T_D.dtype == torch.float32
        with torch.autocast(x_B_T_H_W_D.device.type, dtype=torch.float32):
            shift, scale = self._modulation(emb_B_T_D, adaln_lora_B_T_3D).chunk(2, dim=-1)
            n = self.layer_norm(x_B_T_H_W_D.float()) * (1 + scale[:, :, None, None, :]) + shift[:, :, None, None, :]
            return self.linear(n)

    def forward(self, x_B_T_H_W_D, emb_B_T_D, adaln_lora_B_T_3D: Optional[torch.Tensor] = None):
        if self.use_wan_fp32_strategy:
            return self._forward_fp32(x_B_T_H_W_D, emb_B_T_D, adaln_lora_B_T_3D)
        shift, scale = self._modulation(emb_B_T_D, adaln_lora_B_T_3D).chunk(2, dim=-1)
        D = x_B_T_H_W_D.shape[-1]
        if not torch.is_grad_enabled() and x_B_T_H_W_D.is_cuda:
            n, _ = ops.ln_modulate(x_B_T_H_W_D, shift.reshape(-1, D), scale.reshape(-1, D), eps=self.layer_norm.eps)
        else:
            n = self.layer_norm(x_B_T_H_W_D) * (1 + scale[:, :, None, None, :].type_as(x_B_T_H_W_D)) + shift[:, :, None, None, :].type_as(x_B_T_H_W_D)
        return self.linear(n)

    @torch.no_grad()
    def forward_jvp(self, x, tx, emb, temb, lora=None, tlora=None):
        f = (lambda e, l: self._modulation(e, l)) if self.use_adaln_lora else (lambda e, l: self._modulation(e, None))
        if lora is None:
            lora = emb.new_zeros(())
        temb = torch.zeros_like(emb) if temb is None else temb
        tlora = torch.zeros_like(lora) if tlora is None else tlora
        if self.use_wan_fp32_strategy:     # a handful of fp32 passes over [B, T, H, W, D], once per network call
            g = lambda x_, e, l: self._forward_fp32(x_, e, l if self.use_adaln_lora else None)
            return torch.func.jvp(g, (x.float(), emb, lora), (tx.float(), temb, tlora))
        m, tm = torch.func.jvp(f, (emb, lora), (temb, tlora))
        D = x.shape[-1]
        (shift, scale), (tshift, tscale) = (z.type_as(x).chunk(2, dim=-1) for z in (m, tm))
        n, tn = ops.stacked_pair(x.shape, x.dtype, x.device)
        ops.ln_modulate(x, shift.reshape(-1, D), scale.reshape(-1, D), tx, tshift.reshape(-1, D), tscale.reshape(-1, D),
                        eps=self.layer_norm.eps, out=n, tout=tn)
        y = self.linear(ops.as_stacked(n, tn))
        b = x.shape[0]
        return y[:b], y[b:]


class _BlockRecompute(torch.autograd.Function):
    """Activation checkpoint of one block that keeps the attention results: the forward pass runs the block without
    autograd and keeps its inputs plus (o, log-sum-exp) of its attention calls (0.7 GB per block at the 2B 720p shape, where
    the forward attention kernels are 85 % of the block); the backward pass runs the block again with autograd,
    taking those results instead of launching the forward kernels, and back-propagates through it.  The reference's
    selective modes make the same choice with a dispatcher policy (:181-198, :1660-1686).  Restriction of this kind of
    checkpoint: use ``loss.backward()`` (``torch.autograd.grad`` with respect to parameters inside does not see them)."""

    @staticmethod
    def forward(ctx, block, x, emb, ctx_text, ctx_img, rope, lora, extra):
        # the second run must compute what the first one did: nothing random inside, same autocast setting
        if block.training and any(isinstance(m, nn.Dropout) and m.p > 0 for m in block.modules()):
            raise NotImplementedError("block checkpointing with active dropout (the recomputation would draw another mask)")
        kept = []
        context = ctx_text if ctx_img is None else (ctx_text, ctx_img)
        with torch.no_grad(), record_attention_results(kept):
            out = block(x, emb, context, rope, lora, extra)
        ctx.block, ctx.kept = block, kept
        ctx.autocast = (torch.is_autocast_enabled("cuda"), torch.get_autocast_dtype("cuda"))
        # saved through autograd's own mechanism: an in-place change of an input before the backward pass is an error,
        # not a silently wrong gradient
        ctx.save_for_backward(x, emb, ctx_text, ctx_img, rope, lora, extra)
        ctx.needs = tuple(t is not None and t.requires_grad for t in (x, emb, ctx_text, ctx_img, rope, lora, extra))
        return out

    @staticmethod
    def backward(ctx, gout):
        ins = [None if t is None else t.detach().requires_grad_(need) for t, need in zip(ctx.saved_tensors, ctx.needs)]
        x, emb, ctx_text, ctx_img, rope, lora, extra = ins
        context = ctx_text if ctx_img is None else (ctx_text, ctx_img)
        enabled, dtype = ctx.autocast
        with torch.enable_grad(), torch.autocast("cuda", enabled=enabled, dtype=dtype), replay_attention_results(ctx.kept):
            out = ctx.block(x, emb, context, rope, lora, extra)
        torch.autograd.backward(out, gout)
        return (None,) + tuple(None if t is None else t.grad for t in ins)


def _checkpoint_every(sac_config) -> int:
    """Activation checkpointing of the blocks, from the reference's ``sac_config`` (a ``SACConfig``-like object or a dict
    with ``mode`` and ``every_n_blocks``; :1660-1686).  0 = off (``None`` or mode "none"); n = every n-th block is
    checkpointed (``_BlockRecompute``).  The reference's modes choose which intermediate results of a block to keep (a
    torch dispatcher policy); here every mode keeps the same ones: the block's inputs and its attention results."""
    if sac_config is None:
        return 0
    get = (lambda k, d: sac_config.get(k, d)) if isinstance(sac_config, dict) else (lambda k, d: getattr(sac_config, k, d))
    mode = get("mode", "none")
    mode = str(getattr(mode, "value", getattr(mode, "name", mode))).lower()
    if mode in ("none", "checkpointmode.none"):
        return 0
    return max(1, int(get("every_n_blocks", 1)))


class MiniTrainDIT(nn.Module):
    def __init__(
        self,
        max_img_h: int,
        max_img_w: int,
        max_frames: int,
        in_channels: int,
        out_channels: int,
        patch_spatial: int,
        patch_temporal: int,
        concat_padding_mask: bool = True,
        model_channels: int = 768,
        num_blocks: int = 10,
        num_heads: int = 16,
        mlp_ratio: float = 4.0,
        atten_backend: str = "hip",
        crossattn_emb_channels: int = 1024,
        use_crossattn_projection: bool = False,
        crossattn_proj_in_channels: int = 1024,
        extra_image_context_dim: Optional[int] = None,
        pos_emb_cls: str = "rope3d",
        pos_emb_learnable: bool = False,
        pos_emb_interpolation: str = "crop",
        min_fps: int = 1,
        max_fps: int = 30,
        use_adaln_lora: bool = False,
        adaln_lora_dim: int = 256,
        rope_h_extrapolation_ratio: float = 1.0,
        rope_w_extrapolation_ratio: float = 1.0,
        rope_t_extrapolation_ratio: float = 1.0,
        extra_per_block_abs_pos_emb: bool = False,
        extra_h_extrapolation_ratio: float = 1.0,
        extra_w_extrapolation_ratio: float = 1.0,
        extra_t_extrapolation_ratio: float = 1.0,
        rope_enable_fps_modulation: bool = True,
        sac_config=None,
        n_dense_blocks: int = -1,
        natten_parameters=None,
        use_wan_fp32_strategy: bool = False,
    ) -> None:
        super().__init__()
        if n_dense_blocks != -1 or natten_parameters is not None:
            raise NotImplementedError("sparse (neighbourhood) attention is not built")
        if pos_emb_cls != "rope3d":
            raise ValueError(f"Unknown pos_emb_cls {pos_emb_cls}")
        self._checkpoint_every = _checkpoint_every(sac_config)
        self.max_img_h, self.max_img_w, self.max_frames = max_img_h, max_img_w, max_frames
        self.in_channels, self.out_channels = in_channels, out_channels
        self.patch_spatial, self.patch_temporal = patch_spatial, patch_temporal
        self.num_heads, self.num_blocks, self.model_channels = num_heads, num_blocks, model_channels
        self.concat_padding_mask = concat_padding_mask
        self.atten_backend = atten_backend
        self.pos_emb_cls = pos_emb_cls
        self.extra_per_block_abs_pos_emb = extra_per_block_abs_pos_emb
        self.extra_image_context_dim = extra_image_context_dim
        self.use_adaln_lora, self.adaln_lora_dim = use_adaln_lora, adaln_lora_dim
        self.use_crossattn_projection = use_crossattn_projection
        self.use_wan_fp32_strategy = use_wan_fp32_strategy

        self.x_embedder = PatchEmbed(patch_spatial, patch_temporal, in_channels + 1 if concat_padding_mask else in_channels, model_channels)
        kwargs = dict(
            model_channels=model_channels, len_h=max_img_h // patch_spatial, len_w=max_img_w // patch_spatial,
            len_t=max_frames // patch_temporal, max_fps=max_fps, min_fps=min_fps, is_learnable=pos_emb_learnable,
            interpolation=pos_emb_interpolation, head_dim=model_channels // num_heads,
            h_extrapolation_ratio=rope_h_extrapolation_ratio, w_extrapolation_ratio=rope_w_extrapolation_ratio,
            t_extrapolation_ratio=rope_t_extrapolation_ratio, enable_fps_modulation=rope_enable_fps_modulation,
        )
        self.pos_embedder = VideoRopePosition3DEmb(**kwargs)
        if extra_per_block_abs_pos_emb:
            kwargs.update(h_extrapolation_ratio=extra_h_extrapolation_ratio, w_extrapolation_ratio=extra_w_extrapolation_ratio,
                          t_extrapolation_ratio=extra_t_extrapolation_ratio)
            self.extra_pos_embedder = LearnablePosEmbAxis(**kwargs)
        self.t_embedder = nn.Sequential(Timesteps(model_channels),
                                        TimestepEmbedding(model_channels, model_channels, use_adaln_lora=use_adaln_lora))
        self.blocks = nn.ModuleList([
            Block(x_dim=model_channels, context_dim=crossattn_emb_channels, num_heads=num_heads, mlp_ratio=mlp_ratio,
                  use_adaln_lora=use_adaln_lora, adaln_lora_dim=adaln_lora_dim, backend=atten_backend,
                  image_context_dim=None if extra_image_context_dim is None else model_channels,
                  use_wan_fp32_strategy=use_wan_fp32_strategy)
            for _ in range(num_blocks)
        ])
        self.final_layer = FinalLayer(model_channels, patch_spatial, patch_temporal, out_channels, use_adaln_lora=use_adaln_lora,
                                      adaln_lora_dim=adaln_lora_dim, use_wan_fp32_strategy=use_wan_fp32_strategy)
        self.t_embedding_norm = RMSNormWeight(model_channels, eps=1e-6)
        if extra_image_context_dim is not None:
            self.img_context_proj = nn.Sequential(nn.Linear(extra_image_context_dim, model_channels, bias=True), nn.GELU())
        if use_crossattn_projection:
            self.crossattn_proj = nn.Sequential(nn.Linear(crossattn_proj_in_channels, crossattn_emb_channels, bias=True), nn.GELU())
        self.init_weights()

    def init_weights(self):
        self.x_embedder.init_weights()
        self.pos_embedder.reset_parameters()
        if self.extra_per_block_abs_pos_emb:
            self.extra_pos_embedder.reset_parameters()
        self.t_embedder[1].init_weights()
        for block in self.blocks:
            block.init_weights()
        self.final_layer.init_weights()
        self.t_embedding_norm.reset_parameters()
        if self.extra_image_context_dim is not None:
            self.img_context_proj[0].reset_parameters()

    # ------------------------------------------------------------------ pieces
    def _with_padding_mask(self, x_B_C_T_H_W, padding_mask):
        """The padding mask, resized (nearest) to the frame size, as one more input channel (:1541-1547)."""
        if not self.concat_padding_mask:
            return x_B_C_T_H_W
        pm = F.interpolate(padding_mask.float(), size=list(x_B_C_T_H_W.shape[-2:]), mode="nearest").to(x_B_C_T_H_W.dtype)
        return torch.cat([x_B_C_T_H_W, pm.unsqueeze(1).repeat(1, 1, x_B_C_T_H_W.shape[2], 1, 1)], dim=1)

    def prepare_embedded_sequence(self, x_B_C_T_H_W, fps=None, padding_mask=None):
        x_B_T_H_W_D = self.x_embedder(self._with_padding_mask(x_B_C_T_H_W, padding_mask))
        extra_pos_emb = self.extra_pos_embedder(x_B_T_H_W_D, fps=fps) if self.extra_per_block_abs_pos_emb else None
        return x_B_T_H_W_D, self.pos_embedder(x_B_T_H_W_D, fps=fps), extra_pos_emb

    def unpatchify(self, x_B_T_H_W_M):
        """``B T H W (p1 p2 t C) -> B C (T t) (H p1) (W p2)`` (:1562-1570)."""
        B, T, H, W, _ = x_B_T_H_W_M.shape
        p, t = self.patch_spatial, self.patch_temporal
        x = x_B_T_H_W_M.reshape(B, T, H, W, p, p, t, self.out_channels)
        return x.permute(0, 7, 1, 6, 2, 4, 3, 5).reshape(B, self.out_channels, T * t, H * p, W * p)

    def _context(self, crossattn_emb, img_context_emb):
        if self.use_crossattn_projection:
            crossattn_emb = self.crossattn_proj(crossattn_emb)
        if img_context_emb is not None:
            assert self.extra_image_context_dim is not None, "extra_image_context_dim must be set if img_context_emb is provided"
            return (crossattn_emb, self.img_context_proj(img_context_emb))
        return crossattn_emb

    def _time_embedding(self, timesteps_B_T):
        """(:1610-1614) under use_wan_fp32_strategy an fp32 autocast region: with fp32 timesteps the embedding, its MLP
        and the RMSNorm stay in fp32."""
        with torch.autocast(timesteps_B_T.device.type, enabled=self.use_wan_fp32_strategy, dtype=torch.float32):
            emb, lora = self.t_embedder(timesteps_B_T)
            return self.t_embedding_norm(emb), lora

    # ------------------------------------------------------------------ the reference's surface
    def forward(self, x_B_C_T_H_W, timesteps_B_T, crossattn_emb, fps=None, padding_mask=None, data_type=None,
                intermediate_feature_ids=None, img_context_emb=None):
        del data_type
        x, rope, extra = self.prepare_embedded_sequence(x_B_C_T_H_W, fps=fps, padding_mask=padding_mask)
        context_input = self._context(crossattn_emb, img_context_emb)
        if timesteps_B_T.ndim == 1:
            timesteps_B_T = timesteps_B_T.unsqueeze(1)
        emb, lora = self._time_embedding(timesteps_B_T)
        feats = []
        recompute = self._checkpoint_every > 0 and torch.is_grad_enabled()
        for i, block in enumerate(self.blocks):
            text, img = context_input if isinstance(context_input, tuple) else (context_input, None)
            # (a checkpoint whose inputs carry no gradient would never be asked to run its backward pass)
            if recompute and i % self._checkpoint_every == 0 and any(
                    t is not None and t.requires_grad for t in (x, emb, text, img, lora, extra)):
                x = _BlockRecompute.apply(block, x, emb, text, img, rope, lora, extra)
            else:
                x = block(x, emb, context_input, rope_emb_L_1_1_D=rope, adaln_lora_B_T_3D=lora, extra_per_block_pos_emb=extra)
            if intermediate_feature_ids and i in intermediate_feature_ids:
                feats.append(x.reshape(x.shape[0], -1, x.shape[-1]))
        out = self.unpatchify(self.final_layer(x, emb, adaln_lora_B_T_3D=lora))
        return (out, feats) if intermediate_feature_ids else out

    # ------------------------------------------------------------------ parallelism hooks of the reference (:1688-1737)
    def enable_context_parallel(self, process_group=None):
        """A group of one rank is accepted (nothing to exchange); more ranks need a second GPU and are refused."""
        self.pos_embedder.enable_context_parallel(process_group=process_group)
        ranks = None
        if process_group is not None:
            import torch.distributed as dist

            ranks = dist.get_process_group_ranks(process_group)
        for block in self.blocks:
            block.set_context_parallel_group(process_group=process_group, ranks=ranks, stream=None)
        self._is_context_parallel_enabled = True

    def disable_context_parallel(self):
        self.pos_embedder.disable_context_parallel()
        for block in self.blocks:
            block.set_context_parallel_group(process_group=None, ranks=None, stream=None)
        self._is_context_parallel_enabled = False

    @property
    def is_context_parallel_enabled(self):
        return getattr(self, "_is_context_parallel_enabled", False)

    def fully_shard(self, mesh):
        raise NotImplementedError("parameter sharding across GPUs (FSDP) is not part of this one-GPU build")

    # ------------------------------------------------------------------ forward mode
    @torch.no_grad()
    def forward_jvp(self, x_B_C_T_H_W, tx_B_C_T_H_W, timesteps_B_T, ttimesteps_B_T, crossattn_emb, fps=None, padding_mask=None,
                    img_context_emb=None) -> Tuple[torch.Tensor, torch.Tensor]:
        """``(out, tout)``: the network output and its derivative along ``(tx, ttimesteps)``.  ``ttimesteps_B_T=None``
        keeps the time fixed."""
        assert tx_B_C_T_H_W.shape == x_B_C_T_H_W.shape
        B = x_B_C_T_H_W.shape[0]
        xin = self._with_padding_mask(x_B_C_T_H_W, padding_mask)
        txin = tx_B_C_T_H_W
        if self.concat_padding_mask:   # the mask channel does not move
            txin = torch.cat([tx_B_C_T_H_W, torch.zeros_like(xin[:, -1:])], dim=1)
        both = self.x_embedder(torch.cat([xin, txin], dim=0))
        x, tx = both[:B], both[B:]
        rope = self.pos_embedder(x, fps=fps)
        extra = self.extra_pos_embedder(x, fps=fps) if self.extra_per_block_abs_pos_emb else None
        context_input = self._context(crossattn_emb, img_context_emb)
        if timesteps_B_T.ndim == 1:
            timesteps_B_T = timesteps_B_T.unsqueeze(1)
        if ttimesteps_B_T is None:
            ttimesteps_B_T = torch.zeros_like(timesteps_B_T)
        elif ttimesteps_B_T.ndim == 1:
            ttimesteps_B_T = ttimesteps_B_T.unsqueeze(1)
        if self.use_adaln_lora:
            (emb, lora), (temb, tlora) = torch.func.jvp(self._time_embedding, (timesteps_B_T,), (ttimesteps_B_T,))
        else:
            emb, temb = torch.func.jvp(lambda t: self._time_embedding(t)[0], (timesteps_B_T,), (ttimesteps_B_T,))
            lora = tlora = None
        for block in self.blocks:
            x, tx = block.forward_jvp(x, tx, emb, temb, context_input, rope, lora, tlora, extra_per_block_pos_emb=extra)
        y, ty = self.final_layer.forward_jvp(x, tx, emb, temb, lora, tlora)
        return self.unpatchify(y), self.unpatchify(ty)


def _is_video(data_type) -> bool:
    """The reference passes a ``DataType`` enum (VIDEO / IMAGE); its name or a plain string is accepted here."""
    if data_type is None:
        return True
    return str(getattr(data_type, "name", data_type)).lower() == "video"


class MinimalV1LVGDiT(MiniTrainDIT):
    """Video-conditioned network (networks/minimal_v1_lvg_dit.py:24-62): the condition mask ``[B, 1, T, H, W]`` (1 on the
    given frames) is one more input channel, zeros for image batches; timesteps are multiplied by ``timestep_scale``."""

    def __init__(self, *args, timestep_scale: float = 1.0, **kwargs):
        assert "in_channels" in kwargs, "in_channels must be provided"
        kwargs["in_channels"] += 1
        self.timestep_scale = timestep_scale
        super().__init__(*args, **kwargs)

    def _with_condition_mask(self, x_B_C_T_H_W, mask, data_type):
        if _is_video(data_type):
            return torch.cat([x_B_C_T_H_W, mask.type_as(x_B_C_T_H_W)], dim=1)
        return torch.cat([x_B_C_T_H_W, torch.zeros_like(x_B_C_T_H_W[:, :1])], dim=1)

    def forward(self, x_B_C_T_H_W, timesteps_B_T, crossattn_emb, condition_video_input_mask_B_C_T_H_W=None, fps=None,
                padding_mask=None, data_type=None, intermediate_feature_ids=None, img_context_emb=None, **kwargs):
        del kwargs
        x = self._with_condition_mask(x_B_C_T_H_W, condition_video_input_mask_B_C_T_H_W, data_type)
        return super().forward(x, timesteps_B_T * self.timestep_scale, crossattn_emb, fps=fps, padding_mask=padding_mask,
                               intermediate_feature_ids=intermediate_feature_ids, img_context_emb=img_context_emb)

    @torch.no_grad()
    def forward_jvp(self, x_B_C_T_H_W, tx_B_C_T_H_W, timesteps_B_T, ttimesteps_B_T, crossattn_emb,
                    condition_video_input_mask_B_C_T_H_W=None, fps=None, padding_mask=None, data_type=None, img_context_emb=None):
        x = self._with_condition_mask(x_B_C_T_H_W, condition_video_input_mask_B_C_T_H_W, data_type)
        tx = torch.cat([tx_B_C_T_H_W, torch.zeros_like(tx_B_C_T_H_W[:, :1])], dim=1)     # the mask does not move
        tts = None if ttimesteps_B_T is None else ttimesteps_B_T * self.timestep_scale
        return super().forward_jvp(x, tx, timesteps_B_T * self.timestep_scale, tts, crossattn_emb, fps=fps,
                                   padding_mask=padding_mask, img_context_emb=img_context_emb)
