"""The DiT ``Attention`` module with ``backend="hip"``: projections (library GEMMs), fused RMSNorm + RoPE and the
attention kernels of this package, with a forward that also carries a tangent.

Reference: ``Attention`` in cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:286-440 -- same constructor
arguments, sub-module and parameter names (``q_proj``, ``k_proj``, ``v_proj``, ``output_proj``, ``q_norm.weight``,
``k_norm.weight``: a reference checkpoint's state dict for the module loads as is), ``init_weights``,
``compute_qkv``, ``compute_attention``, ``forward``, ``set_context_parallel_group``.  What the reference selects
with ``backend`` in :361-375 is fixed to the HIP op here.

``forward_jvp`` has no counterpart in the reference checkout: its JVP attention kernel
(utils/flash_attention_jvp_triton.py) ships without the caller that pushes a tangent through the surrounding
layers.  The rule used here is the plain one: linear layers map the tangent with the same weights (primal and tangent
go through each GEMM stacked along the batch), RMSNorm + RoPE and attention use their fused JVP kernels.

Reverse mode: ``forward`` is differentiable end to end -- the projections through torch, RMSNorm + RoPE through
``cosmos_norm_rope_bwd`` and the attention through ``cosmos_attn_bwd``.  ``forward_jvp`` runs without autograd (the
tangent pass of the distillation recipes is taken under ``no_grad``).
"""
from __future__ import annotations

import math
import weakref
from typing import Optional, Tuple

import torch
from torch import nn

from . import ops
from .attention import results_are_kept
from .attn_op import HipAttnOp


class HeadRMSNormWeight(nn.Module):
    """Holds the ``weight`` of a per-head RMSNorm (``te.pytorch.RMSNorm(head_dim, eps=1e-6)``, minimal_v4_dit.py:350-353);
    the arithmetic happens in the fused kernel."""

    def __init__(self, head_dim: int, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(head_dim))

    def reset_parameters(self) -> None:
        nn.init.ones_(self.weight)


class _NormRopeFn(torch.autograd.Function):
    """Fused RMSNorm + RoPE with its reverse-mode rule (heads-first output memory, ``[B, S, H, D]`` view)."""

    @staticmethod
    def forward(ctx, x, weight, rope_emb, eps):
        y, _ = ops.norm_rope(x, weight, rope_emb, None, eps=eps, out_layout="bhsd")
        ctx.save_for_backward(x, weight, rope_emb if rope_emb is not None else x.new_empty(0))
        ctx.has_rope, ctx.eps = rope_emb is not None, eps
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, rope_emb = ctx.saved_tensors
        dx, dweight = ops.norm_rope_bwd(x, weight, rope_emb if ctx.has_rope else None, dy, eps=ctx.eps,
                                        need_dweight=ctx.needs_input_grad[1])
        return dx, (None if dweight is None else dweight.to(weight.dtype)), None, None


class Attention(nn.Module):
    def __init__(
        self,
        query_dim: int,
        context_dim=None,
        n_heads=8,
        head_dim=64,
        dropout=0.0,
        qkv_format: str = "bshd",
        backend: str = "hip",
        use_wan_fp32_strategy: bool = False,
    ) -> None:
        super().__init__()
        self.is_selfattn = context_dim is None
        # "minimal_a2a" is the reference's name for the op protocol that HipAttnOp implements (a2a_cp.py:208-219): configurations
        # written for the reference keep working.  Other libraries' kernels ("torch", "transformer_engine", ...) are not here.
        assert backend in ["hip", "minimal_a2a"], f"Invalid backend: {backend}"
        assert qkv_format == "bshd", "only the bshd format of the DiT is built"
        # use_wan_fp32_strategy (minimal_v4_dit.py:410-412) lifts the 16-bit RMSNorm output of q, k to fp32 for the rotation;
        # the attention call then casts the result to 16 bits.  The fused RMSNorm + RoPE kernel has exactly these rounding
        # points with or without the flag (16-bit normalised value, fp32 rotation, one rounding at the store): the flag
        # changes nothing here.
        self.backend = backend
        context_dim = query_dim if context_dim is None else context_dim
        inner_dim = head_dim * n_heads
        self.n_heads = n_heads
        self.head_dim = head_dim
        self.qkv_format = qkv_format
        self.query_dim = query_dim
        self.context_dim = context_dim
        self.use_wan_fp32_strategy = use_wan_fp32_strategy

        self.q_proj = nn.Linear(query_dim, inner_dim, bias=False)
        self.q_norm = HeadRMSNormWeight(head_dim, eps=1e-6)
        self.k_proj = nn.Linear(context_dim, inner_dim, bias=False)
        self.k_norm = HeadRMSNormWeight(head_dim, eps=1e-6)
        self.v_proj = nn.Linear(context_dim, inner_dim, bias=False)
        self.v_norm = nn.Identity()
        self.output_proj = nn.Linear(inner_dim, query_dim, bias=False)
        self.output_dropout = nn.Dropout(dropout) if dropout > 1e-4 else nn.Identity()
        self.attn_op = HipAttnOp()
        # Cross-attention against a context that does not change between calls (the text conditioning over the steps of a
        # sampler, or over the two passes of a JVP): its projected, normalised and re-tiled keys and values are kept per
        # context tensor and reused while neither that tensor nor the weights that made them have changed.  Used only where
        # no graph is recorded (inference and forward mode).  ``cache_context = False`` turns it off.
        self.cache_context = True
        self._context_cache = {}

        self._query_dim = query_dim
        self._context_dim = context_dim
        self._inner_dim = inner_dim

    def init_weights(self) -> None:
        """Same initialisation as minimal_v4_dit.py:381-393: truncated normal with std 1/sqrt(fan_in), cut at 3 std."""
        for lin, fan_in in ((self.q_proj, self._query_dim), (self.k_proj, self._context_dim),
                            (self.v_proj, self._context_dim), (self.output_proj, self._inner_dim)):
            std = 1.0 / math.sqrt(fan_in)
            torch.nn.init.trunc_normal_(lin.weight, std=std, a=-3 * std, b=3 * std)
        for layer in (self.q_norm, self.k_norm, self.v_norm):
            if hasattr(layer, "reset_parameters"):
                layer.reset_parameters()

    # ------------------------------------------------------------------ pieces
    def _heads(self, t: torch.Tensor) -> torch.Tensor:
        """``b ... (h d) -> b (...) h d`` (minimal_v4_dit.py:400-403), sequence dims flattened for the kernels."""
        return t.reshape(t.shape[0], -1, self.n_heads, self.head_dim)

    @staticmethod
    def _stack(x: torch.Tensor, tx: Optional[torch.Tensor]):
        """Primal and tangent along the batch, so that a linear layer maps both in one GEMM (no copy when the two
        already are the halves of one buffer)."""
        if tx is None:
            return x
        both = ops.as_stacked(x, tx)
        return both if both is not None else torch.cat([x, tx], dim=0)

    @staticmethod
    def _apply_stacked(lin: nn.Linear, xs: torch.Tensor, has_tangent: bool):
        y = lin(xs)
        if not has_tangent:
            return y, None
        b = y.shape[0] // 2
        return y[:b], y[b:]

    def _norm_rope(self, t, norm: HeadRMSNormWeight, rope_emb, tt=None):
        rope = rope_emb if (self.is_selfattn and rope_emb is not None) else None   # only for self-attention (:409)
        if tt is None and torch.is_grad_enabled() and (t.requires_grad or norm.weight.requires_grad):
            return _NormRopeFn.apply(t, norm.weight, rope, norm.eps), None
        return ops.norm_rope(t, norm.weight, rope, tt, eps=norm.eps, out_layout="bhsd")

    def _packed_context(self, slot: str, context: torch.Tensor, k_proj: nn.Linear, k_norm, v_proj: nn.Linear) -> "ops.PackedKV":
        """Keys and values of ``context`` (projection, per-head RMSNorm, no rotation), re-tiled for the kernels.  The entry
        is reused only for the very same tensor object (held by a weak reference, so a new tensor that happens to get the
        freed one's address is never mistaken for it) at the same version, with weights at the same address and version."""
        params = (k_proj.weight, k_norm.weight, v_proj.weight)
        # Inference tensors (made under torch.inference_mode(), as the reference's text encoder makes the context) carry no
        # version counter, so a change in place could not be noticed: those are re-tiled on every call.
        cacheable = self.cache_context and not (context.is_inference() or any(w.is_inference() for w in params))
        key = None
        if cacheable:
            compute_dtype = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled("cuda") else k_proj.weight.dtype
            key = (context._version, tuple(context.shape), context.dtype, context.device, compute_dtype,
                   tuple((w.data_ptr(), w._version, w.dtype) for w in params))
            hit = self._context_cache.get(slot)
            if hit is not None and hit[0]() is context and hit[1] == key:
                return hit[2]
        k, _ = self._norm_rope(self._heads(k_proj(context)), k_norm, None)
        v = self._heads(v_proj(context))
        packed = ops.pack_kv(k.transpose(1, 2), v.transpose(1, 2))
        if cacheable:
            self._context_cache[slot] = (weakref.ref(context), key, packed)
        return packed

    def __getstate__(self):
        state = self.__dict__.copy()
        state["_context_cache"] = {}          # weak references and device images are not part of a copy of the module
        return state

    def _context_is_fixed(self, x: torch.Tensor, context) -> bool:
        if context is None or not isinstance(context, torch.Tensor) or not x.is_cuda:
            return False
        if not isinstance(self.v_norm, nn.Identity) or results_are_kept():
            return False
        # no autograd graph will be built: grad mode off, or nothing on the way requires a gradient
        return not (torch.is_grad_enabled() and (x.requires_grad or context.requires_grad or any(p.requires_grad for p in self.parameters())))

    # ------------------------------------------------------------------ the reference's surface
    def compute_qkv(self, x, context=None, rope_emb=None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """q, k, v as ``[B, S, H, D]`` (q and k in heads-first memory, ready for the kernels)."""
        context = x if context is None else context
        q = self._heads(self.q_proj(x))
        k = self._heads(self.k_proj(context))
        v = self._heads(self.v_norm(self.v_proj(context)))
        q, _ = self._norm_rope(q, self.q_norm, rope_emb)
        k, _ = self._norm_rope(k, self.k_norm, rope_emb)
        return q, k, v

    def compute_attention(self, q, k, v, video_size=None):
        result = self.attn_op(q, k, v, video_size=video_size)   # [B, S, H*D]
        return self.output_dropout(self.output_proj(result))

    def forward(self, x, context: Optional[torch.Tensor] = None, rope_emb: Optional[torch.Tensor] = None, video_size=None):
        """x: ``[B, Mq, K]`` (or ``[B, T, H, W, K]``); context: ``[B, Mk, Kc]`` or None for self-attention; rope_emb: the
        angles ``[Mq, 1, 1, D]`` (self-attention only).  Returns ``[B, Mq, K]`` in the shape of x."""
        if self._context_is_fixed(x, context):
            q, _ = self._norm_rope(self._heads(self.q_proj(x)), self.q_norm, rope_emb)
            packed = self._packed_context("context", context, self.k_proj, self.k_norm, self.v_proj)
            out = self.output_dropout(self.output_proj(self.attn_op.forward_packed(q, packed)))
            return out.reshape(*x.shape[:-1], out.shape[-1])
        q, k, v = self.compute_qkv(x, context, rope_emb=rope_emb)
        out = self.compute_attention(q, k, v, video_size=video_size)
        return out.reshape(*x.shape[:-1], out.shape[-1])

    def set_context_parallel_group(self, process_group, ranks, stream):
        self.attn_op.set_context_parallel_group(process_group, ranks, stream)

    # ------------------------------------------------------------------ forward mode
    @torch.no_grad()
    def forward_jvp(self, x, tx, context=None, tcontext=None, rope_emb=None):
        """``(out, tout)``: the module's output and its directional derivative along ``(tx, tcontext)``.
        ``tcontext=None`` with a context means the context does not move (text conditioning)."""
        assert tx is not None and tx.shape == x.shape
        if isinstance(self.output_dropout, nn.Dropout) and self.training:
            raise NotImplementedError("forward_jvp with active dropout")
        xs = self._stack(x, tx)
        q, tq = self._apply_stacked(self.q_proj, xs, True)
        if tcontext is None and self._context_is_fixed(x, context):
            q, tq = self._norm_rope(self._heads(q), self.q_norm, rope_emb, self._heads(tq))
            packed = self._packed_context("context", context, self.k_proj, self.k_norm, self.v_proj)
            o, to = self.attn_op.forward_packed(q, packed, tq)
            out, tout = self._apply_stacked(self.output_proj, self._stack(o, to), True)
            shape = (*x.shape[:-1], out.shape[-1])
            return out.reshape(shape), tout.reshape(shape)
        if context is None:
            k, tk = self._apply_stacked(self.k_proj, xs, True)
            v, tv = self._apply_stacked(self.v_proj, xs, True)
        else:
            assert tcontext is None or tcontext.shape == context.shape
            cs = self._stack(context, tcontext)
            k, tk = self._apply_stacked(self.k_proj, cs, tcontext is not None)
            v, tv = self._apply_stacked(self.v_proj, cs, tcontext is not None)
        h = self._heads
        q, tq = self._norm_rope(h(q), self.q_norm, rope_emb, h(tq))
        k, tk = self._norm_rope(h(k), self.k_norm, rope_emb, None if tk is None else h(tk))
        o, to = self.attn_op.forward_jvp(q, k, h(v), tq, tk, None if tv is None else h(tv))
        out, tout = self._apply_stacked(self.output_proj, self._stack(o, to), True)
        shape = (*x.shape[:-1], out.shape[-1])
        return out.reshape(shape), tout.reshape(shape)


class I2VCrossAttention(Attention):
    """Cross-attention over a text context and an image context with separate key / value projections, the two results
    summed before the output projection (cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:451-493).  ``context``
    is the pair ``(text_context, img_context)``; parameter names as in the reference (``k_img``, ``v_img``,
    ``k_img_norm``)."""

    def __init__(self, *args, img_latent_dim: int = 1024, **kwargs):
        super().__init__(*args, **kwargs)
        inner_dim = self.head_dim * self.n_heads
        self.k_img = nn.Linear(img_latent_dim, inner_dim, bias=False)
        self.v_img = nn.Linear(img_latent_dim, inner_dim, bias=False)
        self.k_img_norm = HeadRMSNormWeight(self.head_dim, eps=1e-6)

    def init_weights(self) -> None:
        super().init_weights()
        torch.nn.init.trunc_normal_(self.k_img.weight, std=1.0 / math.sqrt(self._inner_dim))
        torch.nn.init.trunc_normal_(self.v_img.weight, std=1.0 / math.sqrt(self._inner_dim))
        self.k_img_norm.reset_parameters()

    def compute_qkv(self, x, context, rope_emb=None):
        text_context, img_context = context
        q, k, v = super().compute_qkv(x, text_context, rope_emb)
        k_img, _ = self._norm_rope(self._heads(self.k_img(img_context)), self.k_img_norm, None)
        v_img = self._heads(self.v_img(img_context))
        return q, k, v, k_img, v_img

    def compute_attention(self, q, k, v, k_img, v_img):
        result = self.attn_op(q, k, v)
        result_img = self.attn_op(q, k_img, v_img)
        return self.output_dropout(self.output_proj(result + result_img))

    def forward(self, x, context=None, rope_emb=None, video_size=None):
        del video_size
        if x.is_cuda and not torch.is_grad_enabled() and not results_are_kept():
            text_context, img_context = context
            q, _ = self._norm_rope(self._heads(self.q_proj(x)), self.q_norm, rope_emb)
            result = self.attn_op.forward_packed(q, self._packed_context("text", text_context, self.k_proj, self.k_norm, self.v_proj))
            result_img = self.attn_op.forward_packed(q, self._packed_context("image", img_context, self.k_img, self.k_img_norm, self.v_img))
            out = self.output_dropout(self.output_proj(result + result_img))
            return out.reshape(*x.shape[:-1], out.shape[-1])
        q, k, v, k_img, v_img = self.compute_qkv(x, context, rope_emb)
        out = self.compute_attention(q, k, v, k_img, v_img)
        return out.reshape(*x.shape[:-1], out.shape[-1])

    @torch.no_grad()
    def forward_jvp(self, x, tx, context=None, tcontext=None, rope_emb=None):
        """``(out, tout)`` along ``tx``; the text and image contexts do not move."""
        assert tcontext is None, "a moving context is not supported by the image-conditioned cross-attention"
        assert tx is not None and tx.shape == x.shape
        text_context, img_context = context
        h = self._heads
        q, tq = self._apply_stacked(self.q_proj, self._stack(x, tx), True)
        q, tq = self._norm_rope(h(q), self.q_norm, rope_emb, h(tq))
        if x.is_cuda:
            o, to = self.attn_op.forward_packed(q, self._packed_context("text", text_context, self.k_proj, self.k_norm, self.v_proj), tq)
            o2, to2 = self.attn_op.forward_packed(q, self._packed_context("image", img_context, self.k_img, self.k_img_norm, self.v_img), tq)
        else:
            k, _ = self._norm_rope(h(self.k_proj(text_context)), self.k_norm, rope_emb)
            k_img, _ = self._norm_rope(h(self.k_img(img_context)), self.k_img_norm, None)
            v, v_img = h(self.v_proj(text_context)), h(self.v_img(img_context))
            o, to = self.attn_op.forward_jvp(q, k, v, tq)
            o2, to2 = self.attn_op.forward_jvp(q, k_img, v_img, tq)
        o.add_(o2)
        to.add_(to2)
        out, tout = self._apply_stacked(self.output_proj, self._stack(o, to), True)
        shape = (*x.shape[:-1], out.shape[-1])
        return out.reshape(shape), tout.reshape(shape)
