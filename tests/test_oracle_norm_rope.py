"""Pins for the CPU oracle of the RMSNorm + rotary step (no GPU).  None of these retypes the closed form:
torch's own rms_norm under forward AD, central finite differences, scalar brute force, and the invariants
that a wrong sign, a wrong pairing (interleaved instead of rotate-half) or a dropped term would break.
"""
import math

import numpy as np
import pytest
import torch


def rnd(shape, seed, std=1.0):
    return np.random.default_rng(seed).standard_normal(shape) * std


def paired_angles(S, D, seed, scale=3.0):
    """Angles with the reference's layout: the half vector repeated twice."""
    half = rnd((S, D // 2), seed, scale)
    return np.concatenate([half, half], axis=-1)


@pytest.mark.parametrize("B,S,H,D", [(1, 7, 3, 16), (2, 5, 2, 32), (1, 3, 5, 64), (1, 4, 1, 128)])
@pytest.mark.parametrize("rope", [True, False])
def test_closed_form_matches_torch_rms_norm_under_jvp(nr_oracle, B, S, H, D, rope):
    x, tx, w = rnd((B, S, H, D), 1), rnd((B, S, H, D), 2, 0.3), 1.0 + 0.2 * rnd((D,), 3)
    a = paired_angles(S, D, 4) if rope else None
    y, ty = nr_oracle.norm_rope_closed_form(x, w, a, tx)
    yt, tyt = nr_oracle.norm_rope_torch(x, w, a, tx)
    np.testing.assert_allclose(y, yt.numpy(), rtol=0, atol=2e-5)
    np.testing.assert_allclose(ty, tyt.numpy(), rtol=0, atol=2e-5)


def test_tangent_matches_central_differences(nr_oracle):
    B, S, H, D = 1, 4, 2, 32
    x, tx, w, a = rnd((B, S, H, D), 5), rnd((B, S, H, D), 6), 1.0 + 0.2 * rnd((D,), 7), paired_angles(S, D, 8)
    _, ty = nr_oracle.norm_rope_closed_form(x, w, a, tx, eps=1e-3)
    h = 1e-6
    yp, _ = nr_oracle.norm_rope_closed_form(x + h * tx, w, a, eps=1e-3)
    ym, _ = nr_oracle.norm_rope_closed_form(x - h * tx, w, a, eps=1e-3)
    np.testing.assert_allclose(ty, (yp - ym) / (2 * h), rtol=0, atol=1e-8)


def test_scalar_brute_force(nr_oracle):
    """Plain loops over one row at a time: mean of squares, divide, then the rotation written pair by pair."""
    B, S, H, D = 1, 3, 2, 16
    x, w, a = rnd((B, S, H, D), 9), 1.0 + 0.2 * rnd((D,), 10), paired_angles(S, D, 11)
    y, _ = nr_oracle.norm_rope_closed_form(x, w, a, eps=1e-6)
    for s in range(S):
        for h in range(H):
            row = x[0, s, h]
            ms = sum(float(v) ** 2 for v in row) / D
            n = [float(row[j]) / math.sqrt(ms + 1e-6) * float(w[j]) for j in range(D)]
            for j in range(D // 2):
                # the pair (j, j + D/2) is rotated by the angle a[s, j] as a 2-D vector
                c, sn = math.cos(a[s, j]), math.sin(a[s, j])
                assert abs(y[0, s, h, j] - (n[j] * c - n[j + D // 2] * sn)) < 1e-12
                assert abs(y[0, s, h, j + D // 2] - (n[j + D // 2] * c + n[j] * sn)) < 1e-12


def test_rotation_invariants(nr_oracle):
    B, S, H, D = 1, 6, 2, 32
    x, w = rnd((B, S, H, D), 12), None
    n, _ = nr_oracle.norm_rope_closed_form(x, w, None)
    # zero angle: identity
    y0, _ = nr_oracle.norm_rope_closed_form(x, w, np.zeros((S, D)))
    np.testing.assert_allclose(y0, n, atol=1e-15)
    # each pair (j, j + D/2) keeps its length (fails for the interleaved pairing or a wrong sign)
    a = paired_angles(S, D, 13)
    y, _ = nr_oracle.norm_rope_closed_form(x, w, a)
    pl = lambda t: t[..., : D // 2] ** 2 + t[..., D // 2 :] ** 2
    np.testing.assert_allclose(pl(y), pl(n), atol=1e-12)
    # quarter turn: (n1, n2) -> (-n2, n1)
    yq, _ = nr_oracle.norm_rope_closed_form(x, w, np.full((S, D), math.pi / 2))
    np.testing.assert_allclose(yq[..., : D // 2], -n[..., D // 2 :], atol=1e-12)
    np.testing.assert_allclose(yq[..., D // 2 :], n[..., : D // 2], atol=1e-12)
    # RMSNorm with unit weight and eps = 0: every row has mean square 1
    n0, _ = nr_oracle.norm_rope_closed_form(x, None, None, eps=0.0)
    np.testing.assert_allclose((n0 ** 2).mean(-1), 1.0, atol=1e-12)


def test_angle_additivity(nr_oracle):
    """Turning by a and then by b is turning by a + b (rows of mean square 1 pass the second RMSNorm unchanged at eps = 0)."""
    S, D = 4, 32
    x, a, b = rnd((1, S, 2, D), 24), paired_angles(S, D, 25), paired_angles(S, D, 26)
    y1, _ = nr_oracle.norm_rope_closed_form(x, None, a, eps=0.0)
    y2, _ = nr_oracle.norm_rope_closed_form(y1, None, b, eps=0.0)
    y12, _ = nr_oracle.norm_rope_closed_form(x, None, a + b, eps=0.0)
    np.testing.assert_allclose(y2, y12, atol=1e-12)


def test_relative_position_property(nr_oracle):
    """<rope(q, m), rope(k, n)> depends on m - n only: angles m * f and n * f for one frequency vector f."""
    D, H = 32, 1
    f = np.abs(rnd((D // 2,), 14))
    f = np.concatenate([f, f])
    q, k = rnd((1, 1, H, D), 15), rnd((1, 1, H, D), 16)

    def dot(m, n):
        yq, _ = nr_oracle.norm_rope_closed_form(q, None, (m * f)[None, :])
        yk, _ = nr_oracle.norm_rope_closed_form(k, None, (n * f)[None, :])
        return float((yq * yk).sum())

    assert abs(dot(3, 1) - dot(10, 8)) < 1e-12
    assert abs(dot(0, 5) - dot(7, 12)) < 1e-12
    assert abs(dot(3, 1) - dot(1, 3)) > 1e-3   # and it does depend on the sign of m - n


def test_rms_norm_invariants(nr_oracle):
    B, S, H, D = 1, 3, 2, 64
    x, tx, w, a = rnd((B, S, H, D), 17), rnd((B, S, H, D), 18), 1.0 + 0.2 * rnd((D,), 19), paired_angles(S, D, 20)
    # scale invariance at eps = 0, and therefore a zero tangent along x itself
    y1, t1 = nr_oracle.norm_rope_closed_form(x, w, a, tx=x, eps=0.0)
    y2, _ = nr_oracle.norm_rope_closed_form(3.7 * x, w, a, eps=0.0)
    np.testing.assert_allclose(y1, y2, atol=1e-12)
    np.testing.assert_allclose(t1, 0.0, atol=1e-12)
    # the tangent is linear in tx
    _, ta = nr_oracle.norm_rope_closed_form(x, w, a, tx=tx)
    _, tb = nr_oracle.norm_rope_closed_form(x, w, a, tx=2.5 * tx + x)
    _, tc = nr_oracle.norm_rope_closed_form(x, w, a, tx=x)
    np.testing.assert_allclose(tb, 2.5 * ta + tc, atol=1e-12)


def test_half_rounding_point(nr_oracle):
    """half= rounds the normalised tensor only: without rotation the result is exactly representable."""
    x = rnd((1, 2, 2, 16), 21)
    n, _ = nr_oracle.norm_rope_closed_form(x, None, None, half="bf16")
    assert np.array_equal(n, torch.from_numpy(n).to(torch.bfloat16).double().numpy())
    nf, _ = nr_oracle.norm_rope_closed_form(x, None, None)
    assert np.abs(n - nf).max() <= 2.0 ** -8 * np.abs(nf).max()


def test_angle_layout_matches_reference_construction(nr_oracle):
    """rope_angles_3d: half vector repeated twice, (t, h, w) blocks of widths dim_t/2, dim_h/2, dim_w/2, position 0 -> 0."""
    T, Hh, W, D = 2, 3, 4, 128
    a = nr_oracle.rope_angles_3d(T, Hh, W, D)
    assert a.shape == (T * Hh * W, D) and a.dtype == np.float32
    assert np.array_equal(a[:, : D // 2], a[:, D // 2 :])
    assert np.all(a[0] == 0)
    dim_h = D // 6 * 2
    dim_t = D - 2 * dim_h
    a4 = a.reshape(T, Hh, W, D)
    # the t block varies with t only, the h block with h only, the w block with w only
    assert np.array_equal(a4[1, 0, 0, : dim_t // 2], a4[1, 2, 3, : dim_t // 2])
    assert np.array_equal(a4[0, 2, 0, dim_t // 2 : dim_t // 2 + dim_h // 2], a4[1, 2, 3, dim_t // 2 : dim_t // 2 + dim_h // 2])
    assert np.array_equal(a4[0, 0, 3, dim_t // 2 + dim_h // 2 : D // 2], a4[1, 2, 3, dim_t // 2 + dim_h // 2 : D // 2])
    # first frequency of every block is 1: the angle equals the coordinate
    assert a4[1, 2, 3, 0] == 1 and a4[1, 2, 3, dim_t // 2] == 2 and a4[1, 2, 3, dim_t // 2 + dim_h // 2] == 3


# ---------------------------------------------------------------- reverse mode
@pytest.mark.parametrize("B,S,H,D", [(1, 5, 3, 16), (2, 4, 2, 64)])
@pytest.mark.parametrize("rope", [True, False])
def test_grads_closed_form_matches_torch_autograd(nr_oracle, B, S, H, D, rope):
    x, dy, w = rnd((B, S, H, D), 31), rnd((B, S, H, D), 32), 1.0 + 0.2 * rnd((D,), 33)
    a = rnd((S, D), 34, 2.0) if rope else None        # arbitrary angles: the two members of a pair may differ
    dx, dw = nr_oracle.norm_rope_grads_closed_form(x, w, a, dy)
    dxt, dwt = nr_oracle.norm_rope_grads_torch(x, w, a, dy, dtype=torch.float64)
    np.testing.assert_allclose(dx, dxt.numpy(), atol=1e-12)
    np.testing.assert_allclose(dw, dwt.numpy(), atol=1e-12)


def test_grads_adjoint_identity_with_the_pinned_jvp(nr_oracle):
    """<dy, J tx> = <J^T dy, tx>, J from the forward-mode closed form pinned above."""
    B, S, H, D = 2, 6, 3, 32
    x, tx, dy, w, a = rnd((B, S, H, D), 35), rnd((B, S, H, D), 36), rnd((B, S, H, D), 37), 1.0 + 0.2 * rnd((D,), 38), paired_angles(S, D, 39)
    _, ty = nr_oracle.norm_rope_closed_form(x, w, a, tx)
    dx, _ = nr_oracle.norm_rope_grads_closed_form(x, w, a, dy)
    assert abs(float((dy * ty).sum()) - float((dx * tx).sum())) < 1e-10


def test_dweight_matches_finite_differences(nr_oracle):
    B, S, H, D = 1, 5, 2, 16
    x, dy, w, a = rnd((B, S, H, D), 40), rnd((B, S, H, D), 41), 1.0 + 0.2 * rnd((D,), 42), paired_angles(S, D, 43)
    _, dw = nr_oracle.norm_rope_grads_closed_form(x, w, a, dy)
    dirw = rnd((D,), 44)
    h = 1e-6
    yp, _ = nr_oracle.norm_rope_closed_form(x, w + h * dirw, a)
    ym, _ = nr_oracle.norm_rope_closed_form(x, w - h * dirw, a)
    assert abs(float((dy * (yp - ym)).sum()) / (2 * h) - float((dw * dirw).sum())) < 1e-7


def test_matches_an_independent_library_implementation(nr_oracle):
    """The rotate-half rotary embedding and the RMSNorm of the `transformers` library (Llama: `apply_rotary_pos_emb`
    with cos / sin tables, `LlamaRMSNorm`) on the same inputs: an implementation written by others, with the same
    non-interleaved pairing that the reference's angle table (half vector repeated twice) is built for."""
    llama = pytest.importorskip("transformers.models.llama.modeling_llama")
    B, S, H, D = 2, 6, 3, 32
    x, w = rnd((B, S, H, D), 41), 1.0 + 0.2 * rnd((D,), 42)
    a = paired_angles(S, D, 43)
    y, _ = nr_oracle.norm_rope_closed_form(x, w, a)
    norm = llama.LlamaRMSNorm(D, eps=1e-6).double()
    with torch.no_grad():
        norm.weight.copy_(torch.from_numpy(w))
        n = norm(torch.from_numpy(x))
        cos, sin = torch.from_numpy(np.cos(a))[None], torch.from_numpy(np.sin(a))[None]     # [1, S, D]
        q, _ = llama.apply_rotary_pos_emb(n, n, cos, sin, unsqueeze_dim=2)                   # [B, S, H, D] layout
    np.testing.assert_allclose(y, q.numpy(), rtol=0, atol=2e-6)     # LlamaRMSNorm computes its statistics in fp32
