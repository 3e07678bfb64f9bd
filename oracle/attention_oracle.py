"""CPU oracle for attention forward + forward-mode JVP (tangent).

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module;
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may use it, and only as the checker (or as the timed CPU baseline),
never as a fallback for the HIP path.

What it restates
----------------
The reference computes this path in a Triton kernel
(``cosmos_predict2/_src/predict2/utils/flash_attention_jvp_triton.py``, below
"JVP") and, forward only, through ``torch.nn.functional.scaled_dot_product_attention``
(``cosmos_predict2/_src/predict2/networks/attention.py:166-180``, below "ATT").
The reference states its own oracle for the JVP kernel in (commented) tests:
naive ``softmax(q k^T s) v`` under ``torch.func.jvp`` (JVP:610-642, JVP:765-812).

Functions
---------
``sdpa_jvp_torch``      torch math-SDPA under ``torch.func.jvp`` in fp32 -- the
                        oracle the tolerance is quoted against.
``closed_form``         numpy fp64 closed form (O, dO, LSE); independent of
                        autograd.  Pinned against ``sdpa_jvp_torch``, finite
                        differences, brute-force loops and invariants in
                        ``tests/test_oracle.py``.
``online_tiles``        numpy restatement of the reference's tile recurrence
                        (JVP:47-153 loop, JVP:299-309 init, JVP:367-378 epilogue)
                        with its rounding points (P and H rounded to the input
                        half type before the P.V-type products, JVP:134-146).
                        Pinned against ``closed_form``.
``sdpa_grads_torch``    torch autograd of math-SDPA in fp32: (dq, dk, dv) for a cotangent
                        of the output -- the oracle of the backward.
``grads_closed_form``   numpy fp64 closed form of the backward.  Pinned against
                        ``sdpa_grads_torch``, finite differences of ``closed_form`` and the
                        adjoint identity <dO, jvp> = <grads, tangents>.
``rows_oracle``         fp32 torch closed form on a block of query rows against
                        the full K/V -- rows are independent, so this is exact
                        and is what large-L parity and the CPU baseline use.
``naive_reference_test_attention``  the reference tests' own oracle function
                        (JVP:620-628) restated, for the tests that re-run the
                        reference's known-answer procedures.

Parity status: every function here is pinned by a check that does not retype its
own formula (see tests/test_oracle.py).  No reference-held golden vectors exist
for this path (the reference's JVP tests are commented-out procedures, not
stored data), so the pins are: torch autograd forward AD, central finite
differences in fp64, brute-force scalar loops on tiny shapes, and invariants.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import numpy as np

LOG2E = 1.4426950408889634
LN2 = 0.6931471805599453


# --------------------------------------------------------------------------- #
# torch: math SDPA under forward-mode AD (the quoted oracle)
# --------------------------------------------------------------------------- #
def _key_padding_mask(key_lens, Lkv, torch):
    if key_lens is None:
        return None
    kl = torch.as_tensor(key_lens, dtype=torch.int64)
    # [B,1,1,Lkv] boolean, True = attend
    return (torch.arange(Lkv)[None, :] < kl[:, None])[:, None, None, :]


def sdpa_jvp_torch(q, k, v, tq=None, tk=None, tv=None, sm_scale=None, causal=False, key_lens=None):
    """(O, dO) = jvp of math scaled_dot_product_attention, fp32 on CPU.

    q,k,v (+ tangents): torch tensors [B,H,L,d] (any float dtype; upcast to fp32
    without changing the values).  Missing tangents are zeros.  ``key_lens``
    ([B] ints) is a key-padding mask: keys >= key_lens[b] are not attended.
    The MATH backend is forced: the fused CPU kernel has no forward-AD formula.
    Mirrors the reference oracle JVP:620-634 and the SDPA call ATT:170-178.
    """
    import torch
    import torch.nn.functional as F
    from torch.nn.attention import SDPBackend, sdpa_kernel

    q, k, v = (x.detach().to("cpu", torch.float32) for x in (q, k, v))
    zeros = lambda x: torch.zeros_like(x)
    tq = zeros(q) if tq is None else tq.detach().to("cpu", torch.float32)
    tk = zeros(k) if tk is None else tk.detach().to("cpu", torch.float32)
    tv = zeros(v) if tv is None else tv.detach().to("cpu", torch.float32)
    mask = _key_padding_mask(key_lens, k.shape[-2], torch)
    assert not (causal and mask is not None)

    def f(q_, k_, v_):
        return F.scaled_dot_product_attention(q_, k_, v_, attn_mask=mask, is_causal=causal, scale=sm_scale)

    with sdpa_kernel(SDPBackend.MATH):
        o, to = torch.func.jvp(f, (q, k, v), (tq, tk, tv))
    return o, to


def sdpa_forward_torch(q, k, v, sm_scale=None, causal=False, key_lens=None):
    """Forward-only math SDPA in fp32 on CPU (ATT:170-178)."""
    import torch
    import torch.nn.functional as F
    from torch.nn.attention import SDPBackend, sdpa_kernel

    q, k, v = (x.detach().to("cpu", torch.float32) for x in (q, k, v))
    mask = _key_padding_mask(key_lens, k.shape[-2], torch)
    with sdpa_kernel(SDPBackend.MATH):
        return F.scaled_dot_product_attention(q, k, v, attn_mask=mask, is_causal=causal, scale=sm_scale)


def naive_reference_test_attention(q, k, v, sm_scale, causal=False):
    """The oracle function of the reference's own (commented) tests, JVP:620-628:
    ``p = softmax((q k^T * s).float()).to(dtype); out = p @ v`` -- in the input dtype."""
    import torch

    p = torch.matmul(q, k.transpose(2, 3)) * sm_scale
    if causal:
        L = q.shape[-2]
        keep = torch.tril(torch.ones((L, L), device=q.device))
        p = p.masked_fill(keep == 0, float("-inf"))
    p = torch.softmax(p.float(), dim=-1).to(q.dtype)
    return torch.matmul(p, v)


# --------------------------------------------------------------------------- #
# numpy fp64 closed form
# --------------------------------------------------------------------------- #
def _np64(x):
    if x is None:
        return None
    if hasattr(x, "detach"):
        import torch

        x = x.detach().to("cpu", torch.float64).numpy()
    return np.asarray(x, dtype=np.float64)


def _valid_mask(B, Lq, Lkv, causal, key_lens):
    """[B,1,Lq,Lkv] boolean, True = attend; or None."""
    m = None
    if causal:
        m = (np.arange(Lkv)[None, :] <= np.arange(Lq)[:, None])[None, None]
        m = np.broadcast_to(m, (B, 1, Lq, Lkv))
    if key_lens is not None:
        kl = np.asarray(key_lens, dtype=np.int64).reshape(B)
        km = (np.arange(Lkv)[None, :] < kl[:, None])[:, None, None, :]
        km = np.broadcast_to(km, (B, 1, Lq, Lkv))
        m = km if m is None else (m & km)
    return m


def closed_form(q, k, v, tq=None, tk=None, tv=None, sm_scale=None, causal=False, key_lens=None):
    """fp64 closed form.  Returns (O, dO, LSE) as numpy float64.

        S  = (Q K^T) s  (-inf where masked)      P = softmax(S)      O = P V
        dS = (dQ K^T + Q dK^T) s                 H = P * dS          r = rowsum(H)
        dO = P dV + H V - r O                    LSE = logsumexp(S)  (natural log, scaled scores)

    The LSE convention follows the reference epilogue JVP:367,376
    (``m += log2(l)``, stored as ``m * ln 2`` with m in the log2 domain of the scaled scores).
    """
    q, k, v, tq, tk, tv = (_np64(x) for x in (q, k, v, tq, tk, tv))
    B, H, Lq, d = q.shape
    Lkv = k.shape[2]
    s = (1.0 / math.sqrt(d)) if sm_scale is None else float(sm_scale)
    S = np.einsum("bhqd,bhkd->bhqk", q, k) * s
    mask = _valid_mask(B, Lq, Lkv, causal, key_lens)
    if mask is not None:
        S = np.where(mask, S, -np.inf)
    m = S.max(axis=-1, keepdims=True)
    E = np.exp(S - m)
    l = E.sum(axis=-1, keepdims=True)
    P = E / l
    O = np.einsum("bhqk,bhkd->bhqd", P, v)
    lse = (m + np.log(l))[..., 0]
    dS = np.zeros_like(S)
    if tq is not None:
        dS = dS + np.einsum("bhqd,bhkd->bhqk", tq, k)
    if tk is not None:
        dS = dS + np.einsum("bhqd,bhkd->bhqk", q, tk)
    dS = dS * s
    Hm = P * dS
    r = Hm.sum(axis=-1, keepdims=True)
    dO = np.einsum("bhqk,bhkd->bhqd", Hm, v) - r * O
    if tv is not None:
        dO = dO + np.einsum("bhqk,bhkd->bhqd", P, tv)
    return O, dO, lse


def sdpa_grads_torch(q, k, v, dout, sm_scale=None, causal=False):
    """(dq, dk, dv) = reverse-mode gradients of math scaled_dot_product_attention w.r.t. q, k, v for the output
    cotangent ``dout``, fp32 on CPU (torch autograd).  The oracle the backward tolerance is quoted against; what the
    reference obtains from flash-attn in ``_attention.backward`` (JVP:505-561) and checks against autograd of naive
    attention in its own procedure (JVP:567-607).
    """
    import torch
    import torch.nn.functional as F
    from torch.nn.attention import SDPBackend, sdpa_kernel

    q, k, v = (x.detach().to("cpu", torch.float32).requires_grad_(True) for x in (q, k, v))
    dout = dout.detach().to("cpu", torch.float32)
    with sdpa_kernel(SDPBackend.MATH):
        o = F.scaled_dot_product_attention(q, k, v, is_causal=causal, scale=sm_scale)
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), dout)
    return dq, dk, dv


def grads_closed_form(q, k, v, dout, sm_scale=None, causal=False):
    """fp64 closed form of the backward.  Returns (dQ, dK, dV) as numpy float64.

        P = softmax(Q K^T s)      dP = dO V^T      D = rowsum(dO * O)      dS = P * (dP - D)
        dV = P^T dO               dK = s dS^T Q    dQ = s dS K

    (the recurrences flash-attn implements for JVP:514-531; D is the usual rowsum(P * dP) rewritten with O = P V).
    """
    q, k, v, dout = (_np64(x) for x in (q, k, v, dout))
    B, H, Lq, d = q.shape
    Lkv = k.shape[2]
    s = (1.0 / math.sqrt(d)) if sm_scale is None else float(sm_scale)
    S = np.einsum("bhqd,bhkd->bhqk", q, k) * s
    mask = _valid_mask(B, Lq, Lkv, causal, None)
    if mask is not None:
        S = np.where(mask, S, -np.inf)
    m = S.max(axis=-1, keepdims=True)
    E = np.exp(S - m)
    P = E / E.sum(axis=-1, keepdims=True)
    O = np.einsum("bhqk,bhkd->bhqd", P, v)
    dP = np.einsum("bhqd,bhkd->bhqk", dout, v)
    D = (dout * O).sum(axis=-1, keepdims=True)
    dS = P * (dP - D)
    dV = np.einsum("bhqk,bhqd->bhkd", P, dout)
    dK = np.einsum("bhqk,bhqd->bhkd", dS, q) * s
    dQ = np.einsum("bhqk,bhkd->bhqd", dS, k) * s
    return dQ, dK, dV


# --------------------------------------------------------------------------- #
# numpy restatement of the reference's online tile recurrence
# --------------------------------------------------------------------------- #
def _round_half(x: np.ndarray, half: Optional[str]) -> np.ndarray:
    """Round fp32/fp64 values to bf16 / fp16 (round-to-nearest-even) and return float64."""
    if half is None:
        return x
    import torch

    dt = {"bf16": torch.bfloat16, "fp16": torch.float16}[half]
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(dt).to(torch.float64).numpy()


def online_tiles(q, k, v, tq, tk, tv, sm_scale=None, causal=False, block_m=64, block_n=32, half: Optional[str] = None):
    """Tile-by-tile restatement of the reference kernel for ONE (batch, head):
    q,tq [Lq,d]; k,tk [Lkv,d]; v,tv [Lkv,dv].  Returns (O, dO, LSE) float64.

    Follows JVP:86-152 (loop), JVP:299-309 (init), JVP:367-378 (epilogue):
    state (m, l, r, acc, acc_A, acc_B) per query row; per KV tile
      qk = q k^T;  tS = (tq k^T + q tk^T) s                          JVP:93-97
      m' = max(m, rowmax(qk) * s*log2e);  p = exp2(qk*s*log2e - m')  JVP:104-105,111
      tail: qk -> -inf, tS -> 0 for keys >= Lkv                      JVP:107-113
      l <- l a + sum p;  H = p*tS;  r <- r a + sum H;  a = exp2(m-m') JVP:112-119
      acc <- acc a + p v;  acc_A <- acc_A a + p tv;  acc_B <- acc_B a + H v   JVP:121-146
      (p and H rounded to the input half type first, JVP:134-143)
    epilogue  O = acc/l;  dO = (acc_A + acc_B - r O)/l;  LSE = (m + log2 l) ln2.
    The causal branch here masks with -inf (the reference adds -1e6, JVP:100;
    the two agree whenever every row keeps at least one key).
    """
    q, k, v, tq, tk, tv = (_np64(x) for x in (q, k, v, tq, tk, tv))
    Lq, d = q.shape
    Lkv, dv = v.shape
    s = (1.0 / math.sqrt(d)) if sm_scale is None else float(sm_scale)
    qk_scale = s * LOG2E
    O = np.zeros((Lq, dv))
    dO = np.zeros((Lq, dv))
    LSE = np.zeros((Lq,))
    for m0 in range(0, Lq, block_m):
        rows = np.arange(m0, min(m0 + block_m, Lq))
        qi, tqi = q[rows], tq[rows]
        m_i = np.full(len(rows), -np.inf)
        l_i = np.zeros(len(rows))
        r_i = np.zeros(len(rows))
        acc = np.zeros((len(rows), dv))
        acc_A = np.zeros((len(rows), dv))
        acc_B = np.zeros((len(rows), dv))
        hi = min(m0 + block_m, Lkv) if causal else Lkv
        for n0 in range(0, hi, block_n):
            cols = np.arange(n0, min(n0 + block_n, Lkv))
            kj, tkj, vj, tvj = k[cols], tk[cols], v[cols], tv[cols]
            qk = qi @ kj.T
            tS = (tqi @ kj.T + qi @ tkj.T) * s
            x = qk * qk_scale
            if causal:
                keep = rows[:, None] >= cols[None, :]
                x = np.where(keep, x, -np.inf)
                tS = np.where(keep, tS, 0.0)
            m_ij = np.maximum(m_i, x.max(axis=1))
            p = np.exp2(x - m_ij[:, None])
            l_ij = p.sum(axis=1)
            Hm = p * tS
            r_ij = Hm.sum(axis=1)
            alpha = np.exp2(m_i - m_ij)
            l_i = l_i * alpha + l_ij
            r_i = r_i * alpha + r_ij
            pr, Hr = _round_half(p, half), _round_half(Hm, half)
            acc = acc * alpha[:, None] + pr @ vj
            acc_A = acc_A * alpha[:, None] + pr @ tvj
            acc_B = acc_B * alpha[:, None] + Hr @ vj
            m_i = m_ij
        m_fin = m_i + np.log2(l_i)
        o = acc / l_i[:, None]
        O[rows] = o
        dO[rows] = (acc_A + acc_B - r_i[:, None] * o) / l_i[:, None]
        LSE[rows] = m_fin * LN2
    return O, dO, LSE


# --------------------------------------------------------------------------- #
# torch fp32 row-block oracle for large L
# --------------------------------------------------------------------------- #
def rows_oracle(q_rows, k, v, tq_rows=None, tk=None, tv=None, sm_scale=None, kv_len=None, row_index=None, causal=False):
    """Closed form in fp32 torch on a block of query rows against the full K/V of
    one or more heads.  q_rows/tq_rows: [..., R, d]; k,tk: [..., Lkv, d]; v,tv: [..., Lkv, dv].
    ``kv_len`` keeps keys < kv_len (one int for all leading dims).  ``row_index`` ([R] ints,
    the absolute query positions) is needed with ``causal``.  Returns (O, dO, LSE) fp32 torch.

    Query rows are independent given K,V, so evaluating a row block is exact; this is how
    parity is checked at L=84480 where the full score matrix (457 GB in fp32) cannot exist.
    """
    import torch

    f32 = lambda x: None if x is None else x.detach().to("cpu", torch.float32)
    q_rows, k, v, tq_rows, tk, tv = (f32(x) for x in (q_rows, k, v, tq_rows, tk, tv))
    d = q_rows.shape[-1]
    s = (1.0 / math.sqrt(d)) if sm_scale is None else float(sm_scale)
    if kv_len is not None:
        k, v = k[..., :kv_len, :], v[..., :kv_len, :]
        tk = None if tk is None else tk[..., :kv_len, :]
        tv = None if tv is None else tv[..., :kv_len, :]
    S = (q_rows @ k.transpose(-1, -2)) * s
    if causal:
        keep = torch.as_tensor(row_index)[:, None] >= torch.arange(k.shape[-2])[None, :]
        S = S.masked_fill(~keep, float("-inf"))
    lse = torch.logsumexp(S, dim=-1)
    P = torch.exp(S - lse[..., None])
    O = P @ v
    dS = torch.zeros_like(S)
    if tq_rows is not None:
        dS = dS + tq_rows @ k.transpose(-1, -2)
    if tk is not None:
        dS = dS + q_rows @ tk.transpose(-1, -2)
    Hm = P * (dS * s)
    r = Hm.sum(dim=-1, keepdim=True)
    dO = Hm @ v - r * O
    if tv is not None:
        dO = dO + P @ tv
    return O, dO, lse


def grads_rows_oracle(q_rows, k, v, dout_rows, sm_scale=None):
    """dQ of a block of query rows, fp32 torch on CPU: a row of dQ depends on its own q and dout rows and on the full K, V
    only (P, O, dP, D, dS of that row; closed form of ``grads_closed_form``).  q_rows, dout_rows: [..., R, d]; k, v:
    [..., Lkv, d].  How the backward is checked at L=84480 (pinned against ``grads_closed_form`` in tests/test_oracle.py)."""
    import torch

    f32 = lambda x: x.detach().to("cpu", torch.float32)
    q_rows, k, v, dout_rows = (f32(x) for x in (q_rows, k, v, dout_rows))
    s = (1.0 / math.sqrt(q_rows.shape[-1])) if sm_scale is None else float(sm_scale)
    P = torch.softmax((q_rows @ k.transpose(-1, -2)) * s, dim=-1)
    O = P @ v
    dP = dout_rows @ v.transpose(-1, -2)
    dS = P * (dP - (dout_rows * O).sum(-1, keepdim=True))
    return (dS @ k) * s


def grads_cols_oracle(q, k_cols, v_cols, o, lse, dout, sm_scale=None):
    """(dK, dV) of a block of keys, fp32 torch on CPU, given the forward's results as the backward itself is given them
    (``o`` [..., Lq, d] and the natural-log ``lse`` [..., Lq] of the scaled scores over ALL keys): with them the columns
    P[:, C] = exp(q k_C^T s - lse) need no other key, so dV_C = P_C^T dO and dK_C = s (P_C * (dO v_C^T - D))^T Q cost
    Lq * |C| * d.  q, o, dout: [..., Lq, d]; k_cols, v_cols: [..., C, d].  Pinned against ``grads_closed_form``."""
    import torch

    f32 = lambda x: x.detach().to("cpu", torch.float32)
    q, k_cols, v_cols, o, lse, dout = (f32(x) for x in (q, k_cols, v_cols, o, lse, dout))
    s = (1.0 / math.sqrt(q.shape[-1])) if sm_scale is None else float(sm_scale)
    P = torch.exp((q @ k_cols.transpose(-1, -2)) * s - lse[..., None])
    dS = P * (dout @ v_cols.transpose(-1, -2) - (dout * o).sum(-1, keepdim=True))
    return (dS.transpose(-1, -2) @ q) * s, P.transpose(-1, -2) @ dout


# --------------------------------------------------------------------------- #
# error metrics and synthetic inputs shared by tests / bench / smoke
# --------------------------------------------------------------------------- #
def error_metrics(got, want) -> Tuple[float, float]:
    """(max-abs error, relative-L2 error) of ``got`` against ``want`` in fp64."""
    g, w = _np64(got), _np64(want)
    diff = g - w
    max_abs = float(np.max(np.abs(diff))) if diff.size else 0.0
    denom = float(np.sqrt(np.sum(w * w)))
    rel_l2 = float(np.sqrt(np.sum(diff * diff)) / denom) if denom > 0 else float(np.sqrt(np.sum(diff * diff)))
    return max_abs, rel_l2


def rms_norm_per_head(x, eps=1e-6):
    """x * rsqrt(mean(x^2, -1) + eps): what the DiT applies to q and k per head before
    attention (cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:350-353, :405-408;
    unit weight at initialisation)."""
    import torch

    return x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def make_inputs(shape_q: Sequence[int], shape_kv: Optional[Sequence[int]] = None, seed=0, primal_std=1.0,
                tangent_std=0.1, rms_norm_qk=False, dtype=None, dv: Optional[int] = None):
    """Seeded synthetic (q,k,v,tq,tk,tv) generated in fp32 on CPU, cast once to ``dtype``
    (default bf16) so the oracle and the kernel see identical bits."""
    import torch

    dtype = torch.bfloat16 if dtype is None else dtype
    g = torch.Generator().manual_seed(seed)
    shape_kv = tuple(shape_q) if shape_kv is None else tuple(shape_kv)
    shape_v = shape_kv if dv is None else (*shape_kv[:-1], dv)
    rn = lambda shp, std: torch.randn(*shp, generator=g, dtype=torch.float32) * std
    q, k, v = rn(shape_q, primal_std), rn(shape_kv, primal_std), rn(shape_v, primal_std)
    if rms_norm_qk:
        q, k = rms_norm_per_head(q), rms_norm_per_head(k)
    tq, tk, tv = rn(shape_q, tangent_std), rn(shape_kv, tangent_std), rn(shape_v, tangent_std)
    return tuple(x.to(dtype) for x in (q, k, v, tq, tk, tv))
