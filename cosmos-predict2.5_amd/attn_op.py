"""The ``attn_op`` objects a DiT ``Attention`` module holds, backed by the HIP kernels.

Reference protocol: ``MinimalA2AAttnOp`` (cosmos_predict2/_src/predict2/networks/a2a_cp.py:208-219):
``op(q_B_S_H_D, k_B_S_H_D, v_B_S_H_D, **kwargs) -> [B, S, H*D]`` and
``set_context_parallel_group(process_group, ranks, stream)``; and the functional
``torch_attention_op`` (cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:252-283).
Only the single-GPU branch exists here (a2a_cp.py:189-193): a context-parallel group of size > 1 is refused.
"""
from __future__ import annotations

from typing import Any

import torch

from .attention import attention
from . import ops


def hip_attention_op(q_B_S_H_D, k_B_S_H_D, v_B_S_H_D):
    """Functional form; accepts ``[B, ..., H, D]`` like the reference op and returns ``[B, ..., H*D]``."""
    in_q_shape = q_B_S_H_D.shape
    in_k_shape = k_B_S_H_D.shape
    q = q_B_S_H_D.reshape(in_q_shape[0], -1, in_q_shape[-2], in_q_shape[-1])
    k = k_B_S_H_D.reshape(in_k_shape[0], -1, in_k_shape[-2], in_k_shape[-1])
    v = v_B_S_H_D.reshape(in_k_shape[0], -1, in_k_shape[-2], v_B_S_H_D.shape[-1])
    out = attention(q, k, v, dtype=q.dtype if q.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16)
    return out.reshape(*in_q_shape[:-2], in_q_shape[-2] * v.shape[-1])


class HipAttnOp(torch.nn.Module):
    """Module form with the ``MinimalA2AAttnOp`` surface."""

    def __init__(self, *args, **kwargs):
        del args, kwargs
        super().__init__()
        self.pg = None
        self.stream = None

    def set_context_parallel_group(self, process_group, ranks, stream):
        del ranks
        if process_group is not None:
            import torch.distributed as dist

            if dist.get_world_size(process_group) > 1:
                raise NotImplementedError("context-parallel attention (all-to-all over several GPUs) is not part of this build")
        self.pg = process_group
        self.stream = stream

    def forward(self, query, key, value, *args: Any, **kwargs) -> torch.Tensor:
        del args, kwargs  # e.g. video_size, used only by the sparse (neighbourhood) op in the reference
        # 16-bit inputs keep their type (fp16 stays fp16); anything else is cast to bf16 as in the reference's attention()
        dtype = query.dtype if query.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
        results = attention(query, key, value, dtype=dtype)
        return results.flatten(-2)

    def forward_jvp(self, query, key, value, t_query, t_key=None, t_value=None):
        """Forward + tangent through the same op: inputs ``[B, S, H, D]``; returns (``[B,S,H*D]``, ``[B,S,H*D]``)."""
        tr = lambda x: None if x is None else x.transpose(1, 2)
        o, to, _ = ops.fwd_jvp(tr(query), tr(key), tr(value), tr(t_query), tr(t_key), tr(t_value),
                               out_layout="blhd", need_lse=False)
        return o.transpose(1, 2).flatten(-2), to.transpose(1, 2).flatten(-2)

    def forward_packed(self, query, packed, t_query=None):
        """The op against a packed (key, value) pair (``ops.pack_kv``): query ``[B, S, H, D]``; returns ``[B, S, H*D]``, and the
        tangent along ``t_query`` as well when that is given."""
        tr = lambda x: None if x is None else x.transpose(1, 2)
        o, to, _ = ops.run_packed(tr(query), packed, tr(t_query), out_layout="blhd", need_lse=False)
        o = o.transpose(1, 2).flatten(-2)
        return o if t_query is None else (o, to.transpose(1, 2).flatten(-2))
