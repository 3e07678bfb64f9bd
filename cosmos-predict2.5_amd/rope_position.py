"""The 3-D rotary position table of the DiT: one angle per (token, head channel), which ``ops.norm_rope`` consumes.

Reference: ``VideoRopePosition3DEmb`` (cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:534-661) on top of
``VideoPositionEmb`` (:495-531) -- same keyword arguments, buffers (``seq``, ``dim_spatial_range``,
``dim_temporal_range``), ``forward(x_B_T_H_W_C, fps)`` and ``generate_embeddings(B_T_H_W_C, fps, h_ntk_factor,
w_ntk_factor, t_ntk_factor)``; the result is ``[(T H W), 1, 1, head_dim]`` fp32 with the channel layout
``cat([t, h, w] * 2)`` (:648-658).  Host-side torch code: the table is built once per input size, it is not on the hot
path.  Context parallelism (:500-531, splitting the table across ranks) is refused: this build runs on one GPU.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn


class VideoRopePosition3DEmb(nn.Module):
    def __init__(
        self,
        *,
        head_dim: int,
        len_h: int,
        len_w: int,
        len_t: int,
        base_fps: int = 24,
        h_extrapolation_ratio: float = 1.0,
        w_extrapolation_ratio: float = 1.0,
        t_extrapolation_ratio: float = 1.0,
        enable_fps_modulation: bool = True,
        **kwargs,
    ):
        del kwargs   # accepted for compatibility with the other positional embeddings of the reference
        super().__init__()
        self._cp_group = None
        self.base_fps = base_fps
        self.max_h, self.max_w, self.max_t = len_h, len_w, len_t
        self.enable_fps_modulation = enable_fps_modulation
        # channel split of a head: two spatial blocks of dim // 6 * 2 channels, the rest temporal (42 / 42 / 44 at 128)
        dim_h = head_dim // 6 * 2
        dim_w = dim_h
        dim_t = head_dim - 2 * dim_h
        assert head_dim == dim_h + dim_w + dim_t, f"bad dim: {head_dim} != {dim_h} + {dim_w} + {dim_t}"
        self._dim_h, self._dim_t = dim_h, dim_t
        self.register_buffer("seq", torch.arange(max(len_h, len_w, len_t), dtype=torch.float))
        self.register_buffer("dim_spatial_range", torch.arange(0, dim_h, 2)[: dim_h // 2].float() / dim_h, persistent=True)
        self.register_buffer("dim_temporal_range", torch.arange(0, dim_t, 2)[: dim_t // 2].float() / dim_t, persistent=True)
        # NTK-aware extrapolation: the base 10000 is stretched by ratio ** (dim / (dim - 2))  (:576-578)
        self.h_ntk_factor = h_extrapolation_ratio ** (dim_h / (dim_h - 2))
        self.w_ntk_factor = w_extrapolation_ratio ** (dim_w / (dim_w - 2))
        self.t_ntk_factor = t_extrapolation_ratio ** (dim_t / (dim_t - 2))

    def reset_parameters(self) -> None:
        dev = self.dim_spatial_range.device
        self.seq = torch.arange(max(self.max_h, self.max_w, self.max_t)).float().to(dev)
        self.dim_spatial_range = torch.arange(0, self._dim_h, 2)[: self._dim_h // 2].float().to(dev) / self._dim_h
        self.dim_temporal_range = torch.arange(0, self._dim_t, 2)[: self._dim_t // 2].float().to(dev) / self._dim_t

    def enable_context_parallel(self, process_group):
        if process_group is not None:
            import torch.distributed as dist

            if dist.get_world_size(process_group) > 1:
                raise NotImplementedError("context parallelism (several GPUs) is not part of this build")
        self._cp_group = process_group

    def disable_context_parallel(self):
        self._cp_group = None

    @property
    def seq_dim(self):
        return 0

    def forward(self, x_B_T_H_W_C: torch.Tensor, fps: Optional[torch.Tensor] = None) -> torch.Tensor:
        return self.generate_embeddings(x_B_T_H_W_C.shape, fps=fps)

    def generate_embeddings(
        self,
        B_T_H_W_C,
        fps: Optional[torch.Tensor] = None,
        h_ntk_factor: Optional[float] = None,
        w_ntk_factor: Optional[float] = None,
        t_ntk_factor: Optional[float] = None,
    ) -> torch.Tensor:
        h_ntk_factor = self.h_ntk_factor if h_ntk_factor is None else h_ntk_factor
        w_ntk_factor = self.w_ntk_factor if w_ntk_factor is None else w_ntk_factor
        t_ntk_factor = self.t_ntk_factor if t_ntk_factor is None else t_ntk_factor
        h_freqs = 1.0 / ((10000.0 * h_ntk_factor) ** self.dim_spatial_range.float())
        w_freqs = 1.0 / ((10000.0 * w_ntk_factor) ** self.dim_spatial_range.float())
        t_freqs = 1.0 / ((10000.0 * t_ntk_factor) ** self.dim_temporal_range.float())

        B, T, H, W, _ = B_T_H_W_C
        assert H <= self.max_h and W <= self.max_w, (
            f"Input dimensions (H={H}, W={W}) exceed the maximum dimensions (max_h={self.max_h}, max_w={self.max_w})"
        )
        t_pos = self.seq[:T]
        if self.enable_fps_modulation:
            uniform_fps = (fps is None) or (fps.min() == fps.max())
            assert uniform_fps or B == 1 or T == 1, (
                "For video batch, batch size should be 1 for non-uniform fps. For image batch, T should be 1"
            )
            if fps is None:
                assert T == 1, "T should be 1 for image batch."
            else:
                t_pos = t_pos / fps[:1] * self.base_fps     # frame index rescaled to the base frame rate (:638-640)
        emb_t = torch.outer(t_pos, t_freqs)
        emb_h = torch.outer(self.seq[:H], h_freqs)
        emb_w = torch.outer(self.seq[:W], w_freqs)
        half = torch.cat(
            [
                emb_t[:, None, None, :].expand(T, H, W, -1),
                emb_h[None, :, None, :].expand(T, H, W, -1),
                emb_w[None, None, :, :].expand(T, H, W, -1),
            ],
            dim=-1,
        )
        return torch.cat([half, half], dim=-1).reshape(T * H * W, 1, 1, -1).float()
