"""Host side of the HIP attention forward + JVP: argument checks, workspace, launch.

``fwd_jvp`` is the one function that talks to the C ABI.  It takes heads-first views
``[B, H, L, d]`` (any batch/head/row strides, innermost stride 1), launches on torch's current
stream, never synchronises, and allocates outputs with ``torch.empty`` like the reference wrapper
(cosmos_predict2/_src/predict2/utils/flash_attention_jvp_triton.py:451-455).
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _lib

_DTYPES = {torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_FP16}
SUPPORTED_HEAD_DIMS = (16, 32, 64, 128, 256)   # (attention at 256 runs slower kernels of its own)
FORWARD_HEAD_DIMS = SUPPORTED_HEAD_DIMS
REFERENCE_HEAD_DIMS = (16, 32, 64, 128, 256)  # what the reference accepts (…jvp_triton.py:444-445)


def _kernel_ready(x: torch.Tensor) -> bool:
    """True if the view can be handed to the kernel as is: d stride 1, 16-byte rows and base."""
    return (
        x.stride(-1) == 1
        and x.data_ptr() % 16 == 0
        and all(s % 8 == 0 for s in x.stride()[:-1])
    )


def _prep_pair(x: torch.Tensor, tx: Optional[torch.Tensor]):
    """Primal and tangent must end up with identical strides (the kernel reads both through one set)."""
    if tx is None:
        return (x if _kernel_ready(x) else x.contiguous()), None
    if _kernel_ready(x) and _kernel_ready(tx) and x.stride() == tx.stride():
        return x, tx
    return x.contiguous(), tx.contiguous()


def _strides3(x: torch.Tensor):
    return (ctypes.c_int64 * 3)(x.stride(0), x.stride(1), x.stride(2))


def _alloc_outputs(B, H, Lq, d_v, q, have_tangent, out_layout, need_lse):
    if out_layout == "bhld":
        o = torch.empty((B, H, Lq, d_v), device=q.device, dtype=q.dtype)
        to = torch.empty_like(o) if have_tangent else None
    elif out_layout == "blhd" and have_tangent:
        # o and to as the two halves of one buffer: a following linear layer maps both in one GEMM without a copy
        both = torch.empty((2, B, Lq, H, d_v), device=q.device, dtype=q.dtype)
        o, to = both[0].transpose(1, 2), both[1].transpose(1, 2)
    elif out_layout == "blhd":
        o, to = torch.empty((B, Lq, H, d_v), device=q.device, dtype=q.dtype).transpose(1, 2), None
    else:
        raise ValueError(f"out_layout={out_layout!r}")
    lse = torch.empty((B, H, Lq), device=q.device, dtype=torch.float32) if need_lse else None
    return o, to, lse


def fwd_jvp(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    tq: Optional[torch.Tensor] = None,
    tk: Optional[torch.Tensor] = None,
    tv: Optional[torch.Tensor] = None,
    causal: bool = False,
    sm_scale: Optional[float] = None,
    key_lens: Optional[torch.Tensor] = None,
    out_layout: str = "bhld",
    need_lse: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """(o, to, lse) for q,k,v (+ tangents) given as ``[B, H, L, d]`` views on one GPU.

    Tangents: none (forward only, ``to`` is None), ``tq`` only, or any mix (missing ones are
    treated as zeros).  ``out_layout``: "bhld" -> o is contiguous ``[B,H,Lq,dv]``; "blhd" -> the
    memory is contiguous ``[B,Lq,H,dv]`` and a ``[B,H,Lq,dv]`` view of it is returned.
    ``key_lens``: optional int32 ``[B]`` device tensor, keys >= key_lens[b] are masked.
    """
    assert q.dim() == 4 and k.dim() == 4 and v.dim() == 4, "q, k, v must be [B, H, L, d]"
    assert q.shape[:-2] == k.shape[:-2] and k.shape[:-2] == v.shape[:-2]
    assert k.shape[-2] == v.shape[-2] and q.shape[-1] == k.shape[-1]
    B, H, Lq, d_qk = q.shape
    Lkv, d_v = v.shape[-2], v.shape[-1]
    assert d_qk in REFERENCE_HEAD_DIMS and d_v in REFERENCE_HEAD_DIMS
    if d_qk not in FORWARD_HEAD_DIMS or d_v not in FORWARD_HEAD_DIMS:
        raise NotImplementedError(f"head dims ({d_qk}, {d_v}): the HIP kernels are built for {FORWARD_HEAD_DIMS}")
    assert (Lq == Lkv) or (not causal), "Causal cross-attention is currently not supported."
    if not q.is_cuda:
        raise RuntimeError("cosmos attention (HIP) needs tensors on a GPU; there is no CPU path")
    if q.dtype not in _DTYPES:
        raise NotImplementedError(f"dtype={q.dtype} is not supported (bf16 / fp16)")
    assert k.dtype == q.dtype and v.dtype == q.dtype
    assert k.device == q.device and v.device == q.device
    for t_, x_ in ((tq, q), (tk, k), (tv, v)):
        if t_ is not None:
            assert t_.shape == x_.shape and t_.dtype == x_.dtype and t_.device == x_.device

    have_tangent = any(t_ is not None for t_ in (tq, tk, tv))
    if have_tangent and tq is None:
        tq = torch.zeros_like(q)
    if tk is not None or tv is not None:  # kernels are built for: none / q only / all three
        tk = torch.zeros_like(k) if tk is None else tk
        tv = torch.zeros_like(v) if tv is None else tv
    q, tq = _prep_pair(q, tq)
    k, tk = _prep_pair(k, tk)
    v, tv = _prep_pair(v, tv)

    if sm_scale is None:
        sm_scale = d_qk ** (-0.5)

    o, to, lse = _alloc_outputs(B, H, Lq, d_v, q, have_tangent, out_layout, need_lse)

    if key_lens is not None:
        assert not causal, "key_lens with causal is not supported"
        key_lens = key_lens.to(device=q.device, dtype=torch.int32).contiguous()
        assert key_lens.shape == (B,)

    desc = _lib.AttnDesc()
    desc.abi_version = _lib.ABI_VERSION
    desc.dtype = _DTYPES[q.dtype]
    desc.B, desc.H, desc.Lq, desc.Lkv, desc.d_qk, desc.d_v = B, H, Lq, Lkv, d_qk, d_v
    desc.causal = 1 if causal else 0
    desc.sm_scale = float(sm_scale)
    desc.q, desc.k, desc.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    desc.tq = tq.data_ptr() if tq is not None else None
    desc.tk = tk.data_ptr() if tk is not None else None
    desc.tv = tv.data_ptr() if tv is not None else None
    desc.q_stride, desc.k_stride, desc.v_stride = _strides3(q), _strides3(k), _strides3(v)
    desc.o, desc.to = o.data_ptr(), (to.data_ptr() if to is not None else None)
    desc.o_stride = _strides3(o)
    desc.lse = lse.data_ptr() if lse is not None else None
    desc.key_lens = key_lens.data_ptr() if key_lens is not None else None

    lib = _lib.load_library()
    with torch.cuda.device(q.device):
        ws_bytes = lib.cosmos_attn_workspace_bytes(ctypes.byref(desc))
        if ws_bytes == 0:
            # invalid descriptor: let the launch entry produce the precise status
            _lib.raise_for_status(lib.cosmos_attn_fwd_jvp(ctypes.byref(desc), None, 0, None) or _lib.ST_BAD_ARG)
        workspace = torch.empty(ws_bytes, device=q.device, dtype=torch.uint8)
        stream = torch.cuda.current_stream(q.device).cuda_stream
        status = lib.cosmos_attn_fwd_jvp(ctypes.byref(desc), workspace.data_ptr(), ws_bytes, stream)
    _lib.raise_for_status(status)
    # workspace / converted inputs are freed to torch's caching allocator here; it is stream-ordered on
    # the launch stream, so reuse by later work on this stream is safe.
    return o, to, lse


class PackedKV:
    """The re-tiled image of one (k, v) pair (no tangents), made by :func:`pack_kv` and consumed by :func:`run_packed`:
    for keys and values that stay the same over many calls (the text context of the DiT's cross-attention)."""

    __slots__ = ("image", "B", "H", "Lkv", "d_qk", "d_v", "dtype", "device")

    def __init__(self, image, B, H, Lkv, d_qk, d_v, dtype, device):
        self.image, self.B, self.H, self.Lkv, self.d_qk, self.d_v, self.dtype, self.device = image, B, H, Lkv, d_qk, d_v, dtype, device


def _packed_desc(B, H, Lq, Lkv, d_qk, d_v, dtype, sm_scale):
    desc = _lib.AttnDesc()
    desc.abi_version = _lib.ABI_VERSION
    desc.dtype = _DTYPES[dtype]
    desc.B, desc.H, desc.Lq, desc.Lkv, desc.d_qk, desc.d_v = B, H, Lq, Lkv, d_qk, d_v
    desc.causal = 0
    desc.sm_scale = float(sm_scale)
    desc.tk = desc.tv = None
    return desc


def pack_kv(k: torch.Tensor, v: torch.Tensor) -> PackedKV:
    """Re-tile k, v (``[B, H, Lkv, d]`` views) once (``cosmos_attn_pack_kv``)."""
    assert k.dim() == 4 and v.dim() == 4 and k.shape[:-1] == v.shape[:-1]
    B, H, Lkv, d_qk = k.shape
    d_v = v.shape[-1]
    assert d_qk in REFERENCE_HEAD_DIMS and d_v in REFERENCE_HEAD_DIMS
    if d_qk not in FORWARD_HEAD_DIMS or d_v not in FORWARD_HEAD_DIMS:
        raise NotImplementedError(f"head dims ({d_qk}, {d_v}): the HIP kernels are built for {FORWARD_HEAD_DIMS}")
    if not k.is_cuda:
        raise RuntimeError("cosmos attention (HIP) needs tensors on a GPU; there is no CPU path")
    if k.dtype not in _DTYPES:
        raise NotImplementedError(f"dtype={k.dtype} is not supported (bf16 / fp16)")
    assert v.dtype == k.dtype and v.device == k.device
    k, _ = _prep_pair(k, None)
    v, _ = _prep_pair(v, None)
    desc = _packed_desc(B, H, 1, Lkv, d_qk, d_v, k.dtype, 1.0)
    desc.k, desc.v = k.data_ptr(), v.data_ptr()
    desc.k_stride, desc.v_stride = _strides3(k), _strides3(v)
    # pack_kv does not touch q / o: any valid addresses and strides pass the descriptor checks
    desc.q, desc.o, desc.tq, desc.to, desc.lse, desc.key_lens = k.data_ptr(), k.data_ptr(), None, None, None, None
    desc.q_stride, desc.o_stride = _strides3(k), _strides3(k)
    lib = _lib.load_library()
    with torch.cuda.device(k.device):
        nbytes = lib.cosmos_attn_packed_bytes(ctypes.byref(desc))
        if nbytes == 0:
            _lib.raise_for_status(lib.cosmos_attn_pack_kv(ctypes.byref(desc), None, 0, None) or _lib.ST_BAD_ARG)
        image = torch.empty(nbytes, device=k.device, dtype=torch.uint8)
        status = lib.cosmos_attn_pack_kv(ctypes.byref(desc), image.data_ptr(), nbytes, torch.cuda.current_stream(k.device).cuda_stream)
    _lib.raise_for_status(status)
    return PackedKV(image, B, H, Lkv, d_qk, d_v, k.dtype, k.device)


def run_packed(
    q: torch.Tensor,
    packed: PackedKV,
    tq: Optional[torch.Tensor] = None,
    sm_scale: Optional[float] = None,
    key_lens: Optional[torch.Tensor] = None,
    out_layout: str = "bhld",
    need_lse: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """:func:`fwd_jvp` (forward only, or tangent on q) against a packed (k, v): ``cosmos_attn_run``.  Same results, bit for bit,
    as the one-call form whenever that one does not cut key ranges (it never does with ``key_lens``)."""
    assert q.dim() == 4
    B, H, Lq, d_qk = q.shape
    assert (B, H, d_qk) == (packed.B, packed.H, packed.d_qk) and q.dtype == packed.dtype and q.device == packed.device
    if tq is not None:
        assert tq.shape == q.shape and tq.dtype == q.dtype and tq.device == q.device
    q, tq = _prep_pair(q, tq)
    d_v = packed.d_v
    if sm_scale is None:
        sm_scale = d_qk ** (-0.5)
    o, to, lse = _alloc_outputs(B, H, Lq, d_v, q, tq is not None, out_layout, need_lse)
    if key_lens is not None:
        key_lens = key_lens.to(device=q.device, dtype=torch.int32).contiguous()
        assert key_lens.shape == (B,)
    desc = _packed_desc(B, H, Lq, packed.Lkv, d_qk, d_v, q.dtype, sm_scale)
    desc.q, desc.tq = q.data_ptr(), (tq.data_ptr() if tq is not None else None)
    desc.k = desc.v = packed.image.data_ptr()          # only tested for NULL by cosmos_attn_run
    desc.q_stride = _strides3(q)
    desc.k_stride = desc.v_stride = (ctypes.c_int64 * 3)(packed.H * packed.Lkv * 8, packed.Lkv * 8, 8)
    desc.o, desc.to = o.data_ptr(), (to.data_ptr() if to is not None else None)
    desc.o_stride = _strides3(o)
    desc.lse = lse.data_ptr() if lse is not None else None
    desc.key_lens = key_lens.data_ptr() if key_lens is not None else None
    lib = _lib.load_library()
    with torch.cuda.device(q.device):
        status = lib.cosmos_attn_run(ctypes.byref(desc), packed.image.data_ptr(), packed.image.numel(),
                                     torch.cuda.current_stream(q.device).cuda_stream)
    _lib.raise_for_status(status)
    return o, to, lse


def bwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    o: torch.Tensor,
    lse: torch.Tensor,
    dout: torch.Tensor,
    causal: bool = False,
    sm_scale: Optional[float] = None,
    max_ds_mib: Optional[int] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dq, dk, dv) for the cotangent ``dout`` of o; all tensors ``[B, H, L, d]`` views on one GPU, ``lse`` the
    forward's ``[B, H, Lq]`` fp32.  Mirrors the reference's ``_attention.backward``
    (cosmos_predict2/_src/predict2/utils/flash_attention_jvp_triton.py:505-561): equal head dims only (:507-509),
    outputs allocated like ``torch.empty_like`` of q, k, v (:513).

    ``max_ds_mib``: workspace the call may spend on keeping the 16-bit dS tiles between its two passes (the descriptor's
    field of that name; negative = never).  Default: 32 GiB, but no more than 40 % of the device memory free right now.
    """
    assert q.shape[-1] == k.shape[-1] and k.shape[-1] == v.shape[-1], "Backward not supported with different headdim."
    B, H, Lq, d = q.shape
    Lkv = k.shape[-2]
    assert k.shape == (B, H, Lkv, d) and v.shape == (B, H, Lkv, d)
    assert o.shape == q.shape and dout.shape == q.shape and lse.shape == (B, H, Lq)
    assert d in REFERENCE_HEAD_DIMS
    if d not in FORWARD_HEAD_DIMS:
        raise NotImplementedError(f"head dim {d}: the HIP kernels are built for {FORWARD_HEAD_DIMS}")
    assert (Lq == Lkv) or (not causal), "Causal cross-attention is currently not supported."
    if not q.is_cuda:
        raise RuntimeError("cosmos attention (HIP) needs tensors on a GPU; there is no CPU path")
    if q.dtype not in _DTYPES:
        raise NotImplementedError(f"dtype={q.dtype} is not supported (bf16 / fp16)")
    for x in (k, v, o, dout):
        assert x.dtype == q.dtype and x.device == q.device
    ready = lambda x: x if _kernel_ready(x) else x.contiguous()
    q, k, v, o, dout = (ready(x) for x in (q, k, v, o, dout))
    lse = lse.to(torch.float32).contiguous()
    if sm_scale is None:
        sm_scale = d ** (-0.5)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    if not all(_kernel_ready(x) for x in (dq, dk, dv)):   # empty_like of an exotic view: fall back to plain layouts
        dq, dk, dv = (torch.empty(x.shape, device=x.device, dtype=x.dtype) for x in (q, k, v))

    desc = _lib.AttnBwdDesc()
    desc.abi_version = _lib.ABI_VERSION
    desc.dtype = _DTYPES[q.dtype]
    desc.B, desc.H, desc.Lq, desc.Lkv, desc.d = B, H, Lq, Lkv, d
    desc.causal = 1 if causal else 0
    desc.sm_scale = float(sm_scale)
    if max_ds_mib is None:
        free_bytes, _ = torch.cuda.mem_get_info(q.device)
        max_ds_mib = max(1, min(32 * 1024, int(0.4 * free_bytes) >> 20))
    desc.max_ds_mib = int(max_ds_mib)
    desc.q, desc.k, desc.v, desc.o, desc.dout = (x.data_ptr() for x in (q, k, v, o, dout))
    desc.lse = lse.data_ptr()
    desc.dq, desc.dk, desc.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    desc.q_stride, desc.k_stride, desc.v_stride = _strides3(q), _strides3(k), _strides3(v)
    desc.o_stride, desc.dout_stride = _strides3(o), _strides3(dout)
    desc.dq_stride, desc.dk_stride, desc.dv_stride = _strides3(dq), _strides3(dk), _strides3(dv)

    lib = _lib.load_library()
    with torch.cuda.device(q.device):
        ws_bytes = lib.cosmos_attn_bwd_workspace_bytes(ctypes.byref(desc))
        if ws_bytes == 0:
            _lib.raise_for_status(lib.cosmos_attn_bwd(ctypes.byref(desc), None, 0, None) or _lib.ST_BAD_ARG)
        workspace = torch.empty(ws_bytes, device=q.device, dtype=torch.uint8)
        stream = torch.cuda.current_stream(q.device).cuda_stream
        status = lib.cosmos_attn_bwd(ctypes.byref(desc), workspace.data_ptr(), ws_bytes, stream)
    _lib.raise_for_status(status)
    return dq, dk, dv


def norm_rope(
    x: torch.Tensor,
    weight: Optional[torch.Tensor] = None,
    rope_emb: Optional[torch.Tensor] = None,
    tx: Optional[torch.Tensor] = None,
    eps: float = 1e-6,
    out_layout: str = "bshd",
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Per-head RMSNorm followed by the rotary embedding, and the tangent of both for ``tx``: what the DiT does to q and
    k between the projections and the attention call (cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:405-415).

    ``x`` (and ``tx``): ``[B, S, H, D]`` 16-bit; ``weight``: RMSNorm's ``[D]`` parameter (None = ones);
    ``rope_emb``: the angles ``[S, 1, 1, D]`` / ``[S, D]`` of minimal_v4_dit.py:648-658 (None = no rotation, as for
    cross-attention keys).  Returns ``(y, ty)`` with the shape of ``x``; ``out_layout="bhsd"`` makes the memory
    heads-first (a ``[B, S, H, D]`` view of it is returned), ready for the attention kernels without a transpose.
    """
    assert x.dim() == 4, "x must be [B, S, H, D]"
    B, S, H, D = x.shape
    assert D in REFERENCE_HEAD_DIMS
    if D not in SUPPORTED_HEAD_DIMS:
        raise NotImplementedError(f"head dim {D}: the HIP kernels are built for {SUPPORTED_HEAD_DIMS}")
    if x.dtype not in _DTYPES:
        raise NotImplementedError(f"dtype={x.dtype} is not supported (bf16 / fp16)")
    if tx is not None:
        assert tx.shape == x.shape and tx.dtype == x.dtype and tx.device == x.device
    assert weight is None or weight.shape == (D,)
    assert rope_emb is None or rope_emb.numel() == S * D, "rope_emb must hold one angle per (position, channel)"
    if not x.is_cuda:
        raise RuntimeError("cosmos attention (HIP) needs tensors on a GPU; there is no CPU path")
    x, tx = _prep_pair(x, tx)
    if weight is not None:
        weight = weight.to(device=x.device, dtype=torch.float32).contiguous()
    if rope_emb is not None:
        rope_emb = rope_emb.to(device=x.device, dtype=torch.float32).reshape(S, D).contiguous()
    if out_layout == "bshd":
        y = torch.empty((B, S, H, D), device=x.device, dtype=x.dtype)
    elif out_layout == "bhsd":
        y = torch.empty((B, H, S, D), device=x.device, dtype=x.dtype).transpose(1, 2)
    else:
        raise ValueError(f"out_layout={out_layout!r}")
    ty = torch.empty_like(y) if tx is not None else None

    desc = _lib.NormRopeDesc()
    desc.abi_version = _lib.ABI_VERSION
    desc.dtype = _DTYPES[x.dtype]
    desc.B, desc.S, desc.H, desc.D = B, S, H, D
    desc.eps = float(eps)
    desc.reserved = 0
    desc.x, desc.tx = x.data_ptr(), (tx.data_ptr() if tx is not None else None)
    desc.weight = weight.data_ptr() if weight is not None else None
    desc.angles = rope_emb.data_ptr() if rope_emb is not None else None
    desc.y, desc.ty = y.data_ptr(), (ty.data_ptr() if ty is not None else None)
    desc.x_stride, desc.y_stride = _strides3(x), _strides3(y)
    lib = _lib.load_library()
    with torch.cuda.device(x.device):
        status = lib.cosmos_norm_rope(ctypes.byref(desc), torch.cuda.current_stream(x.device).cuda_stream)
    _lib.raise_for_status(status)
    return y, ty


def norm_rope_bwd(
    x: torch.Tensor,
    weight: Optional[torch.Tensor],
    rope_emb: Optional[torch.Tensor],
    dy: torch.Tensor,
    eps: float = 1e-6,
    need_dweight: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Reverse mode of :func:`norm_rope`: ``(dx, dweight)`` from the gradient ``dy`` of its output.  ``x``, ``dy``:
    ``[B, S, H, D]`` views (any batch / sequence / head strides that are multiples of 8 elements); ``dx`` is contiguous
    ``[B, S, H, D]``; ``dweight`` is fp32 ``[D]`` (None if not wanted).  This is what autograd derives for the RMSNorm and
    rotary ops of cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:405-415."""
    assert x.dim() == 4 and dy.shape == x.shape and dy.dtype == x.dtype and dy.device == x.device
    B, S, H, D = x.shape
    assert D in REFERENCE_HEAD_DIMS
    if D not in SUPPORTED_HEAD_DIMS:
        raise NotImplementedError(f"head dim {D}: the HIP kernels are built for {SUPPORTED_HEAD_DIMS}")
    if x.dtype not in _DTYPES:
        raise NotImplementedError(f"dtype={x.dtype} is not supported (bf16 / fp16)")
    assert weight is None or weight.shape == (D,)
    assert rope_emb is None or rope_emb.numel() == S * D, "rope_emb must hold one angle per (position, channel)"
    if not x.is_cuda:
        raise RuntimeError("cosmos attention (HIP) needs tensors on a GPU; there is no CPU path")
    x = x if _kernel_ready(x) else x.contiguous()
    dy = dy if _kernel_ready(dy) else dy.contiguous()
    if weight is not None:
        weight = weight.to(device=x.device, dtype=torch.float32).contiguous()
    if rope_emb is not None:
        rope_emb = rope_emb.to(device=x.device, dtype=torch.float32).reshape(S, D).contiguous()
    dx = torch.empty((B, S, H, D), device=x.device, dtype=x.dtype)
    dweight = torch.empty((D,), device=x.device, dtype=torch.float32) if need_dweight else None

    desc = _lib.NormRopeBwdDesc()
    desc.abi_version = _lib.ABI_VERSION
    desc.dtype = _DTYPES[x.dtype]
    desc.B, desc.S, desc.H, desc.D = B, S, H, D
    desc.eps = float(eps)
    desc.reserved = 0
    desc.x, desc.dy, desc.dx = x.data_ptr(), dy.data_ptr(), dx.data_ptr()
    desc.weight = weight.data_ptr() if weight is not None else None
    desc.angles = rope_emb.data_ptr() if rope_emb is not None else None
    desc.dweight = dweight.data_ptr() if dweight is not None else None
    desc.x_stride, desc.dy_stride, desc.dx_stride = _strides3(x), _strides3(dy), _strides3(dx)
    lib = _lib.load_library()
    with torch.cuda.device(x.device):
        ws_bytes = lib.cosmos_norm_rope_bwd_workspace_bytes(ctypes.byref(desc))
        workspace = torch.empty(max(ws_bytes, 16), device=x.device, dtype=torch.uint8)
        status = lib.cosmos_norm_rope_bwd(ctypes.byref(desc), workspace.data_ptr(), ws_bytes,
                                          torch.cuda.current_stream(x.device).cuda_stream)
    _lib.raise_for_status(status)
    return dx, dweight


# ------------------------------------------------------------------ elementwise steps of the DiT block (+ tangents)
def stacked_pair(shape, dtype, device):
    """Two tensors of ``shape`` that are the halves of one ``[2, *shape]`` buffer (see :func:`as_stacked`)."""
    both = torch.empty((2, *shape), device=device, dtype=dtype)
    return both[0], both[1]


def as_stacked(x: torch.Tensor, tx: torch.Tensor) -> Optional[torch.Tensor]:
    """If ``x`` and ``tx`` are the two contiguous halves of one buffer, the ``[2 * x.shape[0], ...]`` view of it (no
    copy); otherwise None."""
    if (x.shape == tx.shape and x.dtype == tx.dtype and x.is_contiguous() and tx.is_contiguous() and x.dim() >= 1
            and x._base is not None and x._base is tx._base
            and tx.data_ptr() == x.data_ptr() + x.numel() * x.element_size()):
        both = x._base
        if both.is_contiguous() and both.data_ptr() == x.data_ptr() and both.numel() == 2 * x.numel():
            return both.view(2 * x.shape[0], *x.shape[1:])
    return None


def _dense16(t: torch.Tensor) -> torch.Tensor:
    return t if (t.is_contiguous() and t.data_ptr() % 16 == 0) else t.contiguous()


def _check_elementwise(x: torch.Tensor) -> None:
    if not x.is_cuda:
        raise RuntimeError("cosmos attention (HIP) needs tensors on a GPU; there is no CPU path")
    if x.dtype not in _DTYPES:
        raise NotImplementedError(f"dtype={x.dtype} is not supported (bf16 / fp16)")


def _launch(fn_name: str, desc, device) -> None:
    lib = _lib.load_library()
    with torch.cuda.device(device):
        status = getattr(lib, fn_name)(ctypes.byref(desc), torch.cuda.current_stream(device).cuda_stream)
    _lib.raise_for_status(status)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def ln_modulate(x, shift, scale, tx=None, tshift=None, tscale=None, eps: float = 1e-6, out=None, tout=None):
    """``LayerNorm(x) * (1 + scale) + shift`` over the last dim (no affine parameters) and its tangent, one pass
    (cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:1166-1167).  ``x``: ``[..., D]``; ``shift`` / ``scale``:
    ``[G, D]`` with ``G`` dividing the number of rows (consecutive rows share a vector).  ``out`` / ``tout``: optional
    preallocated outputs (e.g. the two halves of one stacked buffer).  Returns ``(y, ty)``."""
    _check_elementwise(x)
    D = x.shape[-1]
    x = _dense16(x)
    rows = x.numel() // D
    shift, scale = _dense16(shift.to(x.dtype)).reshape(-1, D), _dense16(scale.to(x.dtype)).reshape(-1, D)
    assert shift.shape == scale.shape and rows % shift.shape[0] == 0
    if tx is not None:
        assert tx.shape == x.shape and tx.dtype == x.dtype
        tx = _dense16(tx)
        tshift = None if tshift is None else _dense16(tshift.to(x.dtype)).reshape(-1, D)
        tscale = None if tscale is None else _dense16(tscale.to(x.dtype)).reshape(-1, D)
        assert (tshift is None or tshift.shape == shift.shape) and (tscale is None or tscale.shape == shift.shape)
    y = torch.empty_like(x) if out is None else out
    ty = (torch.empty_like(x) if tout is None else tout) if tx is not None else None
    assert y.is_contiguous() and y.shape == x.shape and (ty is None or (ty.is_contiguous() and ty.shape == x.shape))
    d = _lib.LnModulateDesc()
    d.abi_version, d.dtype = _lib.ABI_VERSION, _DTYPES[x.dtype]
    d.D, d.rows_per_group, d.eps, d.reserved, d.rows = D, rows // shift.shape[0], float(eps), 0, rows
    d.x, d.tx, d.shift, d.scale = _ptr(x), _ptr(tx), _ptr(shift), _ptr(scale)
    d.tshift, d.tscale = (_ptr(tshift), _ptr(tscale)) if tx is not None else (None, None)
    d.y, d.ty = _ptr(y), _ptr(ty)
    _launch("cosmos_ln_modulate", d, x.device)
    return y, ty


def gated_residual(x, res, gate, tx=None, tres=None, tgate=None, inplace: bool = False):
    """``x + gate * res`` and its tangent ``tx + tgate * res + gate * tres`` in one pass
    (cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:1199, :1231, :1241).  ``gate``: ``[G, D]`` as in
    :func:`ln_modulate`.  ``inplace`` overwrites ``x`` / ``tx``.  Returns ``(out, tout)``."""
    _check_elementwise(x)
    D = x.shape[-1]
    assert res.shape == x.shape and res.dtype == x.dtype
    xs, res = _dense16(x), _dense16(res)
    rows = xs.numel() // D
    gate = _dense16(gate.to(x.dtype)).reshape(-1, D)
    assert rows % gate.shape[0] == 0
    if tx is not None:
        assert tres is not None and tx.shape == x.shape and tres.shape == x.shape
        txs, tres = _dense16(tx), _dense16(tres)
        tgate = None if tgate is None else _dense16(tgate.to(x.dtype)).reshape(-1, D)
    else:
        txs = None
    out = xs if (inplace and xs is x) else torch.empty_like(xs)
    tout = None if tx is None else (txs if (inplace and txs is tx) else torch.empty_like(txs))
    d = _lib.GatedResidualDesc()
    d.abi_version, d.dtype = _lib.ABI_VERSION, _DTYPES[x.dtype]
    d.D, d.rows_per_group, d.rows = D, rows // gate.shape[0], rows
    d.x, d.tx, d.res, d.tres = _ptr(xs), _ptr(txs), _ptr(res), (_ptr(tres) if tx is not None else None)
    d.gate, d.tgate = _ptr(gate), (_ptr(tgate) if tx is not None else None)
    d.out, d.tout = _ptr(out), _ptr(tout)
    _launch("cosmos_gated_residual", d, x.device)
    return out, tout


def gelu(h, th=None, inplace: bool = False):
    """Exact (erf) GELU and its tangent ``th * gelu'(h)`` in one pass (``nn.GELU()`` of
    cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:225).  Returns ``(a, ta)``."""
    _check_elementwise(h)
    hs = _dense16(h)
    assert hs.numel() % 8 == 0, "the number of elements must be a multiple of 8"
    ths = None
    if th is not None:
        assert th.shape == h.shape and th.dtype == h.dtype
        ths = _dense16(th)
    a = hs if (inplace and hs is h) else torch.empty_like(hs)
    ta = None if th is None else (ths if (inplace and ths is th) else torch.empty_like(ths))
    d = _lib.GeluDesc()
    d.abi_version, d.dtype, d.n = _lib.ABI_VERSION, _DTYPES[h.dtype], hs.numel()
    d.h, d.th, d.a, d.ta = _ptr(hs), _ptr(ths), _ptr(a), _ptr(ta)
    _launch("cosmos_gelu", d, h.device)
    return a, ta
