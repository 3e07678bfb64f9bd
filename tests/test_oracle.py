"""Pins for the CPU oracle (no GPU).  None of these checks retypes the formula under test:
autograd forward AD, central finite differences, scalar brute force, algebraic invariants, stored vectors.
"""
import math
import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attn_jvp_golden.npz")


def rand64(shape, seed, std=1.0):
    return np.random.default_rng(seed).standard_normal(shape) * std


def make64(B, H, Lq, Lkv, d, dv, seed):
    return (rand64((B, H, Lq, d), seed), rand64((B, H, Lkv, d), seed + 1), rand64((B, H, Lkv, dv), seed + 2),
            rand64((B, H, Lq, d), seed + 3, 0.3), rand64((B, H, Lkv, d), seed + 4, 0.3), rand64((B, H, Lkv, dv), seed + 5, 0.3))


# ---------------------------------------------------------------- closed form vs autograd forward AD
@pytest.mark.parametrize("case", [
    dict(B=1, H=2, Lq=33, Lkv=33, d=16, dv=16),
    dict(B=2, H=1, Lq=17, Lkv=45, d=32, dv=64, key_lens=[45, 9]),
    dict(B=1, H=2, Lq=40, Lkv=40, d=64, dv=64, causal=True),
    dict(B=1, H=1, Lq=5, Lkv=130, d=128, dv=32, sm_scale=0.5),
])
def test_closed_form_matches_torch_sdpa_jvp_fp64(oracle, case):
    c = dict(case)
    causal, key_lens, sm_scale = c.pop("causal", False), c.pop("key_lens", None), c.pop("sm_scale", None)
    q, k, v, tq, tk, tv = make64(seed=3, **c)
    import torch.nn.functional as F
    from torch.nn.attention import SDPBackend, sdpa_kernel

    t = lambda x: torch.from_numpy(x)
    mask = None
    if key_lens is not None:
        mask = (torch.arange(c["Lkv"])[None, :] < torch.tensor(key_lens)[:, None])[:, None, None, :]
    f = lambda a, b, cc: F.scaled_dot_product_attention(a, b, cc, attn_mask=mask, is_causal=causal, scale=sm_scale)
    with sdpa_kernel(SDPBackend.MATH):
        o_ref, to_ref = torch.func.jvp(f, (t(q), t(k), t(v)), (t(tq), t(tk), t(tv)))
    o, to, lse = oracle.closed_form(q, k, v, tq, tk, tv, sm_scale=sm_scale, causal=causal, key_lens=key_lens)
    np.testing.assert_allclose(o, o_ref.numpy(), rtol=0, atol=1e-12)
    np.testing.assert_allclose(to, to_ref.numpy(), rtol=0, atol=1e-12)


def test_sdpa_jvp_wrapper_matches_closed_form_fp32(oracle):
    q, k, v, tq, tk, tv = oracle.make_inputs((2, 2, 50, 64), (2, 2, 70, 64), seed=1, dtype=torch.float32)
    o, to = oracle.sdpa_jvp_torch(q, k, v, tq, tk, tv, key_lens=[70, 13])
    o2, to2, _ = oracle.closed_form(q, k, v, tq, tk, tv, key_lens=[70, 13])
    assert oracle.error_metrics(o, o2)[0] < 2e-6 and oracle.error_metrics(to, to2)[0] < 2e-6
    o, to = oracle.sdpa_jvp_torch(q[..., :50, :], k[..., :50, :], v[..., :50, :], tq, tk[..., :50, :], tv[..., :50, :], causal=True)
    o2, to2, _ = oracle.closed_form(q, k[..., :50, :], v[..., :50, :], tq, tk[..., :50, :], tv[..., :50, :], causal=True)
    assert oracle.error_metrics(o, o2)[0] < 2e-6 and oracle.error_metrics(to, to2)[0] < 2e-6


def test_config1_fp32_plumbing_within_1e5(oracle):
    """The CPU plumbing configuration: B1 H16 L2048 d128 fp32, N(0,1)*0.5, scale 1/sqrt(128): torch math SDPA + jvp (fp32) against
    the fp64 closed form, tolerance 1e-5 (4 heads are checked in fp64 to keep the CPU suite short)."""
    q, k, v, tq, tk, tv = oracle.make_inputs((1, 16, 2048, 128), seed=0, primal_std=0.5, tangent_std=0.5, dtype=torch.float32)
    o, to = oracle.sdpa_jvp_torch(q, k, v, tq, tk, tv)
    sl = slice(3, 16, 4)
    o2, to2, _ = oracle.closed_form(*(x[:, sl] for x in (q, k, v, tq, tk, tv)))
    assert oracle.error_metrics(o[:, sl], o2)[0] <= 1e-5
    assert oracle.error_metrics(to[:, sl], to2)[0] <= 1e-5


# ---------------------------------------------------------------- finite differences and brute force
def test_tangent_matches_central_finite_differences(oracle):
    q, k, v, tq, tk, tv = make64(1, 2, 9, 14, 16, 8, seed=7)
    eps = 1e-6
    op, _, lp = oracle.closed_form(q + eps * tq, k + eps * tk, v + eps * tv)
    om, _, lm = oracle.closed_form(q - eps * tq, k - eps * tk, v - eps * tv)
    _, to, _ = oracle.closed_form(q, k, v, tq, tk, tv)
    np.testing.assert_allclose(to, (op - om) / (2 * eps), rtol=0, atol=2e-8)


def test_brute_force_scalar_loops(oracle):
    B, H, Lq, Lkv, d, dv = 1, 1, 3, 5, 4, 2
    q, k, v, tq, tk, tv = make64(B, H, Lq, Lkv, d, dv, seed=9)
    s = 0.37
    o, to, lse = oracle.closed_form(q, k, v, tq, tk, tv, sm_scale=s)
    for i in range(Lq):
        sc = [s * sum(q[0, 0, i, x] * k[0, 0, j, x] for x in range(d)) for j in range(Lkv)]
        dsc = [s * sum(tq[0, 0, i, x] * k[0, 0, j, x] + q[0, 0, i, x] * tk[0, 0, j, x] for x in range(d)) for j in range(Lkv)]
        z = sum(math.exp(x) for x in sc)
        p = [math.exp(x) / z for x in sc]
        dbar = sum(p[j] * dsc[j] for j in range(Lkv))
        dp = [p[j] * (dsc[j] - dbar) for j in range(Lkv)]          # derivative of softmax
        assert abs(lse[0, 0, i] - math.log(z)) < 1e-12
        for y in range(dv):
            assert abs(o[0, 0, i, y] - sum(p[j] * v[0, 0, j, y] for j in range(Lkv))) < 1e-12
            assert abs(to[0, 0, i, y] - sum(dp[j] * v[0, 0, j, y] + p[j] * tv[0, 0, j, y] for j in range(Lkv))) < 1e-12


# ---------------------------------------------------------------- invariants
def test_invariants(oracle):
    q, k, v, tq, tk, tv = make64(1, 2, 12, 20, 32, 16, seed=21)
    z = lambda x: np.zeros_like(x)
    o, to, lse = oracle.closed_form(q, k, v, tq, tk, tv)
    # linear in the tangent; the q/k/v parts add up
    _, to_q, _ = oracle.closed_form(q, k, v, tq, z(tk), z(tv))
    _, to_k, _ = oracle.closed_form(q, k, v, z(tq), tk, z(tv))
    _, to_v, _ = oracle.closed_form(q, k, v, z(tq), z(tk), tv)
    np.testing.assert_allclose(to, to_q + to_k + to_v, atol=1e-13)
    _, to3, _ = oracle.closed_form(q, k, v, 3 * tq, 3 * tk, 3 * tv)
    np.testing.assert_allclose(to3, 3 * to, atol=1e-12)
    # dQ = dK = 0: the tangent is plain attention applied to dV
    o_dv, _, _ = oracle.closed_form(q, k, tv)
    np.testing.assert_allclose(to_v, o_dv, atol=1e-13)
    # missing tangents mean zeros
    _, to_q2, _ = oracle.closed_form(q, k, v, tq)
    np.testing.assert_allclose(to_q2, to_q, atol=0)
    # V constant along keys: O is that constant and the q/k tangent vanishes
    vc = np.broadcast_to(v[:, :, :1, :], v.shape)
    oc, toc, _ = oracle.closed_form(q, k, vc, tq, tk, z(tv))
    np.testing.assert_allclose(oc, np.broadcast_to(v[:, :, :1, :], oc.shape), atol=1e-13)
    np.testing.assert_allclose(toc, 0, atol=1e-13)
    # a single key: O = V, dO = dV
    o1, to1, _ = oracle.closed_form(q, k[:, :, :1], v[:, :, :1], tq, tk[:, :, :1], tv[:, :, :1])
    np.testing.assert_allclose(o1, np.broadcast_to(v[:, :, :1], o1.shape), atol=1e-13)
    np.testing.assert_allclose(to1, np.broadcast_to(tv[:, :, :1], to1.shape), atol=1e-13)
    # LSE against torch.logsumexp of the scaled scores
    S = torch.from_numpy(np.einsum("bhqd,bhkd->bhqk", q, k) / math.sqrt(q.shape[-1]))
    np.testing.assert_allclose(lse, torch.logsumexp(S, -1).numpy(), atol=1e-12)
    # shifting all keys by a vector c adds q.c to every score of a row: O unchanged
    o_s, _, _ = oracle.closed_form(q, k + 0.25, v)
    np.testing.assert_allclose(o_s, o, atol=1e-12)


def test_key_padding_equals_slicing(oracle):
    q, k, v, tq, tk, tv = make64(2, 2, 7, 30, 16, 16, seed=5)
    lens = [30, 11]
    o, to, lse = oracle.closed_form(q, k, v, tq, tk, tv, key_lens=lens)
    for b, n in enumerate(lens):
        ob, tob, lb = oracle.closed_form(q[b:b + 1], k[b:b + 1, :, :n], v[b:b + 1, :, :n], tq[b:b + 1], tk[b:b + 1, :, :n], tv[b:b + 1, :, :n])
        np.testing.assert_allclose(o[b:b + 1], ob, atol=1e-13)
        np.testing.assert_allclose(to[b:b + 1], tob, atol=1e-13)
        np.testing.assert_allclose(lse[b:b + 1], lb, atol=1e-13)


# ---------------------------------------------------------------- tile recurrence (the reference kernel's algorithm)
@pytest.mark.parametrize("Lq,Lkv,bm,bn,causal", [(70, 70, 64, 32, False), (70, 70, 64, 32, True), (33, 100, 16, 64, False), (128, 15, 128, 16, False)])
def test_online_tiles_matches_closed_form(oracle, Lq, Lkv, bm, bn, causal):
    q, k, v, tq, tk, tv = make64(1, 1, Lq, Lkv, 32, 16, seed=13)
    o, to, lse = oracle.closed_form(q, k, v, tq, tk, tv, sm_scale=0.3, causal=causal)
    o2, to2, lse2 = oracle.online_tiles(q[0, 0], k[0, 0], v[0, 0], tq[0, 0], tk[0, 0], tv[0, 0], sm_scale=0.3, causal=causal, block_m=bm, block_n=bn)
    np.testing.assert_allclose(o2, o[0, 0], atol=1e-12)
    np.testing.assert_allclose(to2, to[0, 0], atol=1e-12)
    np.testing.assert_allclose(lse2, lse[0, 0], atol=1e-12)


def test_online_tiles_with_half_rounding_stays_within_kernel_tolerance(oracle):
    """The reference rounds P and H to the 16-bit input type before the P.V-type products (JVP:134-146); with bf16
    inputs that rounding alone must leave plenty of room inside max-abs 2e-2 / rel-L2 5e-3."""
    q, k, v, tq, tk, tv = (x.double().numpy()[0, 0] for x in oracle.make_inputs((1, 1, 200, 128), seed=2))
    o, to, _ = oracle.closed_form(*(x[None, None] for x in (q, k, v, tq, tk, tv)))
    o2, to2, _ = oracle.online_tiles(q, k, v, tq, tk, tv, block_m=64, block_n=32, half="bf16")
    for got, want in ((o2, o[0, 0]), (to2, to[0, 0])):
        ma, rl = oracle.error_metrics(got, want)
        assert ma < 5e-3 and rl < 3e-3


def test_rows_oracle_matches_closed_form(oracle):
    q, k, v, tq, tk, tv = oracle.make_inputs((1, 2, 300, 64), seed=4, dtype=torch.float32)
    o, to, lse = oracle.closed_form(q, k, v, tq, tk, tv)
    rows = slice(100, 228)
    o2, to2, lse2 = oracle.rows_oracle(q[:, :, rows], k, v, tq[:, :, rows], tk, tv)
    assert oracle.error_metrics(o2, o[:, :, rows])[0] < 2e-6
    assert oracle.error_metrics(to2, to[:, :, rows])[0] < 2e-6
    assert oracle.error_metrics(lse2, lse[:, :, rows])[0] < 2e-6
    o3, to3, _ = oracle.rows_oracle(q[:, :, rows], k, v, tq[:, :, rows], tk, tv, kv_len=77)
    o4, to4, _ = oracle.closed_form(q[:, :, rows], k[:, :, :77], v[:, :, :77], tq[:, :, rows], tk[:, :, :77], tv[:, :, :77])
    assert oracle.error_metrics(o3, o4)[0] < 2e-6 and oracle.error_metrics(to3, to4)[0] < 2e-6
    o5, to5, _ = oracle.rows_oracle(q[:, :, rows], k, v, tq[:, :, rows], tk, tv, causal=True, row_index=list(range(100, 228)))
    o6, to6, _ = oracle.closed_form(q, k, v, tq, tk, tv, causal=True)
    assert oracle.error_metrics(o5, o6[:, :, rows])[0] < 2e-6 and oracle.error_metrics(to5, to6[:, :, rows])[0] < 2e-6


# ---------------------------------------------------------------- the reference's own (commented) known-answer procedures
@pytest.mark.parametrize("shape,causal", [((1, 2, 256, 64), False), ((1, 2, 199, 64), True)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_reference_test_procedure_oracle_agrees(oracle, shape, causal, dtype):
    """flash_attention_jvp_triton.py:610-642 (`_test_jvp`, shapes shortened for CPU): inputs N(0, 0.5), sm_scale 0.5,
    seed 20; the reference's oracle is naive attention (softmax in fp32, cast to dtype) under torch.func.jvp, and its
    tolerance is atol = rtol = 1e-2.  Our fp64 closed form must sit inside that tolerance of the reference's oracle."""
    torch.manual_seed(20)
    mk = lambda: torch.empty(shape, dtype=dtype).normal_(mean=0.0, std=0.5)
    q, k, v, tq, tk, tv = mk(), mk(), mk(), mk(), mk(), mk()
    f = lambda a, b, c: oracle.naive_reference_test_attention(a, b, c, 0.5, causal)
    ref_o, ref_to = torch.func.jvp(f, (q, k, v), (tq, tk, tv))
    o, to, _ = oracle.closed_form(q, k, v, tq, tk, tv, sm_scale=0.5, causal=causal)
    torch.testing.assert_close(torch.from_numpy(o).to(dtype), ref_o, atol=1e-2, rtol=0)
    torch.testing.assert_close(torch.from_numpy(to).to(dtype), ref_to, atol=1e-2, rtol=1e-2)


# ---------------------------------------------------------------- stored vectors
def test_golden_vectors(oracle):
    import importlib.util

    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(os.path.dirname(GOLDEN), "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    gold = np.load(GOLDEN)
    for name in mg.CASES:
        (q, k, v, tq, tk, tv), kw = mg.case_inputs(oracle, name)
        o, to, lse = oracle.closed_form(q, k, v, tq, tk, tv, **kw)
        assert oracle.error_metrics(o, gold[name + "/o"])[0] < 3e-6, name
        assert oracle.error_metrics(to, gold[name + "/to"])[0] < 3e-6, name
        assert oracle.error_metrics(lse, gold[name + "/lse"])[0] < 3e-6, name


def test_error_metrics(oracle):
    a = np.array([1.0, 2.0, 2.0])
    ma, rl = oracle.error_metrics(a + np.array([0.0, 0.3, 0.0]), a)
    assert abs(ma - 0.3) < 1e-12 and abs(rl - 0.1) < 1e-12


# ------------------------------------------------------------------ backward oracle
@pytest.mark.parametrize("causal", [False, True])
def test_grads_closed_form_matches_torch_autograd(oracle, causal):
    import torch

    q, k, v, tq, _, _ = oracle.make_inputs((1, 2, 37, 16), (1, 2, 37 if causal else 53, 16), seed=5, dtype=torch.float64)
    dout = tq[..., : v.shape[-1]].clone()   # any cotangent of the output's shape
    want = oracle.sdpa_grads_torch(q, k, v, dout, sm_scale=0.3, causal=causal)
    got = oracle.grads_closed_form(q, k, v, dout, sm_scale=0.3, causal=causal)
    for g, w in zip(got, want):
        assert np.abs(g - w.double().numpy()).max() < 2e-5   # sdpa_grads_torch computes in fp32


def test_grads_closed_form_is_the_adjoint_of_the_jvp(oracle):
    """<dout, J t> = <J^T dout, t> with the forward-mode closed form (pinned independently) as J."""
    import torch

    q, k, v, tq, tk, tv = oracle.make_inputs((2, 2, 19, 8), (2, 2, 23, 8), seed=9, dtype=torch.float64)
    dout = torch.randn(q.shape[:-1] + (v.shape[-1],), generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    _, jt, _ = oracle.closed_form(q, k, v, tq, tk, tv, sm_scale=0.4)
    dq, dk, dv = oracle.grads_closed_form(q, k, v, dout, sm_scale=0.4)
    lhs = float((dout.numpy() * jt).sum())
    rhs = float((dq * tq.numpy()).sum() + (dk * tk.numpy()).sum() + (dv * tv.numpy()).sum())
    assert abs(lhs - rhs) <= 1e-10 * max(1.0, abs(lhs))


def test_grads_closed_form_matches_finite_differences(oracle):
    import torch

    q, k, v, _, _, _ = oracle.make_inputs((1, 1, 5, 4), (1, 1, 6, 4), seed=2, dtype=torch.float64)
    dout = torch.randn(1, 1, 5, 4, generator=torch.Generator().manual_seed(3), dtype=torch.float64)
    dq, dk, dv = oracle.grads_closed_form(q, k, v, dout, sm_scale=0.5)
    loss = lambda q_, k_, v_: float((oracle.closed_form(q_, k_, v_, sm_scale=0.5)[0] * dout.numpy()).sum())
    eps = 1e-6
    for name, x, g in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        for idx in [(0, 0, 0, 0), (0, 0, 2, 3), (0, 0, 4, 1)]:
            xp, xm = x.clone(), x.clone()
            xp[idx] += eps; xm[idx] -= eps
            args_p = {"q": (xp, k, v), "k": (q, xp, v), "v": (q, k, xp)}[name]
            args_m = {"q": (xm, k, v), "k": (q, xm, v), "v": (q, k, xm)}[name]
            fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(fd - g[idx]) < 1e-6, (name, idx, fd, g[idx])


def test_grads_rows_and_cols_oracles_match_closed_form(oracle):
    """The row-block (dQ) and key-block (dK, dV) oracles used at L=84480 equal the full fp64 closed form on the rows / keys
    they cover; the key-block oracle takes the forward's o and lse as inputs, as the backward kernels do."""
    q, k, v, tq, _, _ = oracle.make_inputs((2, 2, 200, 32), (2, 2, 150, 32), seed=11, dtype=torch.float32)
    dout = tq * 7.0
    dq, dk, dv = oracle.grads_closed_form(q, k, v, dout, sm_scale=0.21)
    o, _, lse = oracle.closed_form(q, k, v, sm_scale=0.21)
    rows, cols = slice(40, 168), slice(90, 150)
    got = oracle.grads_rows_oracle(q[:, :, rows], k, v, dout[:, :, rows], sm_scale=0.21)
    assert oracle.error_metrics(got, dq[:, :, rows])[1] < 1e-5
    gk, gv = oracle.grads_cols_oracle(q, k[:, :, cols], v[:, :, cols], torch.from_numpy(o), torch.from_numpy(lse), dout, sm_scale=0.21)
    assert oracle.error_metrics(gk, dk[:, :, cols])[1] < 1e-5 and oracle.error_metrics(gv, dv[:, :, cols])[1] < 1e-5
    # a wrong lse (e.g. base-2, or of unscaled scores) or a dropped D term must fail: the check has teeth
    bad_k, bad_v = oracle.grads_cols_oracle(q, k[:, :, cols], v[:, :, cols], torch.from_numpy(o), torch.from_numpy(lse) * 1.4427, dout, sm_scale=0.21)
    assert oracle.error_metrics(bad_v, dv[:, :, cols])[1] > 1e-2
    bad_k, _ = oracle.grads_cols_oracle(q, k[:, :, cols], v[:, :, cols], torch.zeros_like(torch.from_numpy(o)), torch.from_numpy(lse), dout, sm_scale=0.21)
    assert oracle.error_metrics(bad_k, dk[:, :, cols])[1] > 1e-2
