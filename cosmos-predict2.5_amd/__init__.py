"""MI355X-native flash-attention forward + forward-mode JVP (and backward) for Cosmos-Predict2.5's DiT attention.

The directory name is not a Python identifier; load it with ``__graft_entry__.load_package()``
(registers it as ``cosmos_predict2_5_amd``).
"""
from . import _lib  # noqa: F401
from .attention import attention as attention_forward
from .attn_op import HipAttnOp, hip_attention_op
from .dit_attention import Attention, I2VCrossAttention
from .dit_block import Block, GPT2FeedForward
from .dit_network import FinalLayer, MinimalV1LVGDiT, MiniTrainDIT, PatchEmbed, TimestepEmbedding, Timesteps
from .flash_attention_jvp import attention as attention_jvp
from .flash_attention_jvp import attention_with_lse
from .rope_position import VideoRopePosition3DEmb
from .ops import PackedKV, bwd, fwd_jvp, gated_residual, gelu, ln_modulate, norm_rope, norm_rope_bwd, pack_kv, run_packed

__all__ = ["attention_jvp", "attention_with_lse", "attention_forward", "HipAttnOp", "hip_attention_op", "fwd_jvp", "pack_kv", "run_packed", "PackedKV", "bwd", "norm_rope", "norm_rope_bwd", "ln_modulate", "gated_residual", "gelu", "Attention", "I2VCrossAttention", "Block", "GPT2FeedForward", "MiniTrainDIT", "MinimalV1LVGDiT", "FinalLayer", "PatchEmbed", "TimestepEmbedding", "Timesteps", "VideoRopePosition3DEmb"]
