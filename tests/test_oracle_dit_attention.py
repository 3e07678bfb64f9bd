"""Pins for the CPU oracle of the DiT Attention module (no GPU): the torch function under forward AD against the
composition of the separately pinned fp64 closed forms with numpy matmuls, and against central finite differences."""
import numpy as np
import pytest
import torch


def make_weights(K, Kc, H, D, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    return {
        "q_proj.weight": r(H * D, K) / K ** 0.5, "k_proj.weight": r(H * D, Kc) / Kc ** 0.5,
        "v_proj.weight": r(H * D, Kc) / Kc ** 0.5, "output_proj.weight": r(K, H * D) / (H * D) ** 0.5,
        "q_norm.weight": 1 + 0.2 * r(D), "k_norm.weight": 1 + 0.2 * r(D),
    }


def composed_fp64(oracle, nr_oracle, w, x, context, angles, H, D, tx, tcontext):
    """The module as a chain of the pinned pieces, fp64 numpy."""
    n = lambda t: None if t is None else t.numpy()
    wq, wk, wv, wo = (w[k].numpy() for k in ("q_proj.weight", "k_proj.weight", "v_proj.weight", "output_proj.weight"))
    x, context, tx, tcontext = n(x), n(context), n(tx), n(tcontext)
    selfattn = context is None
    c, tc = (x, tx) if selfattn else (context, tcontext)
    hd = lambda t: None if t is None else t.reshape(t.shape[0], -1, H, D)
    lin = lambda t, m: None if t is None else t @ m.T
    ang = angles if selfattn else None
    q, tq = nr_oracle.norm_rope_closed_form(hd(lin(x, wq)), w["q_norm.weight"].numpy(), ang, hd(lin(tx, wq)))
    k, tk = nr_oracle.norm_rope_closed_form(hd(lin(c, wk)), w["k_norm.weight"].numpy(), ang, hd(lin(tc, wk)))
    v, tv = hd(lin(c, wv)), hd(lin(tc, wv))
    sw = lambda t: None if t is None else np.ascontiguousarray(np.swapaxes(t, 1, 2))
    o, to, _ = oracle.closed_form(sw(q), sw(k), sw(v), sw(tq), sw(tk), sw(tv))
    fl = lambda t: np.swapaxes(t, 1, 2).reshape(t.shape[0], t.shape[2], H * D)
    return fl(o) @ wo.T, fl(to) @ wo.T


@pytest.mark.parametrize("cross,moving_context", [(False, False), (True, False), (True, True)])
def test_module_oracle_matches_composition_of_pinned_pieces(oracle, nr_oracle, dit_oracle, cross, moving_context):
    B, Mq, Mk, K, Kc, H, D = 2, 12, 7, 24, 20, 3, 16
    g = torch.Generator().manual_seed(1)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    w = make_weights(K, Kc if cross else K, H, D, 2)
    x, tx = r(B, Mq, K), r(B, Mq, K) * 0.3
    context = r(B, Mk, Kc) if cross else None
    tcontext = r(B, Mk, Kc) * 0.3 if (cross and moving_context) else None
    half = np.random.default_rng(3).standard_normal((Mq, D // 2)) * 2
    angles = np.concatenate([half, half], -1)
    out, tout = dit_oracle.attention_module_torch(w, x, context, angles, H, D, tx, tcontext, dtype=torch.float64)
    want, twant = composed_fp64(oracle, nr_oracle, w, x, context, angles, H, D, tx, tcontext)
    np.testing.assert_allclose(out.numpy(), want, atol=1e-10)
    np.testing.assert_allclose(tout.numpy(), twant, atol=1e-10)


def test_module_oracle_tangent_matches_central_differences(dit_oracle):
    B, Mq, K, H, D = 1, 9, 16, 2, 16
    g = torch.Generator().manual_seed(4)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    w = make_weights(K, K, H, D, 5)
    x, tx = r(B, Mq, K), r(B, Mq, K)
    half = np.random.default_rng(6).standard_normal((Mq, D // 2))
    angles = np.concatenate([half, half], -1)
    f = lambda x_: dit_oracle.attention_module_torch(w, x_, None, angles, H, D, dtype=torch.float64)[0]
    _, tout = dit_oracle.attention_module_torch(w, x, None, angles, H, D, tx, dtype=torch.float64)
    h = 1e-6
    np.testing.assert_allclose(tout.numpy(), ((f(x + h * tx) - f(x - h * tx)) / (2 * h)).numpy(), atol=1e-7)


def test_rope_is_skipped_for_cross_attention(dit_oracle):
    """minimal_v4_dit.py:409: the rotation applies to self-attention only."""
    B, Mq, Mk, K, H, D = 1, 5, 4, 16, 2, 16
    g = torch.Generator().manual_seed(7)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    w = make_weights(K, K, H, D, 8)
    x, c = r(B, Mq, K), r(B, Mk, K)
    a = np.ones((Mq, D))
    o1, _ = dit_oracle.attention_module_torch(w, x, c, a, H, D, dtype=torch.float64)
    o2, _ = dit_oracle.attention_module_torch(w, x, c, None, H, D, dtype=torch.float64)
    assert torch.equal(o1, o2)


def test_module_grads_adjoint_identity_and_weight_finite_differences(dit_oracle):
    B, Mq, K, H, D = 1, 9, 16, 2, 16
    g = torch.Generator().manual_seed(21)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    w = make_weights(K, K, H, D, 22)
    x, tx, dout = r(B, Mq, K), r(B, Mq, K), r(B, Mq, K)
    half = np.random.default_rng(23).standard_normal((Mq, D // 2))
    angles = np.concatenate([half, half], -1)
    grads = dit_oracle.attention_module_grads_torch(w, x, dout, None, angles, H, D, dtype=torch.float64)
    # <dout, J tx> = <J^T dout, tx> with J from forward mode (pinned above)
    _, tout = dit_oracle.attention_module_torch(w, x, None, angles, H, D, tx, dtype=torch.float64)
    assert abs(float((dout * tout).sum()) - float((grads["x"] * tx).sum())) < 1e-9
    # one random direction in every weight, central differences of <dout, out>
    h = 1e-6
    for name in w:
        dirw = r(*w[name].shape)
        wp, wm = dict(w), dict(w)
        wp[name], wm[name] = w[name] + h * dirw, w[name] - h * dirw
        fp = dit_oracle.attention_module_torch(wp, x, None, angles, H, D, dtype=torch.float64)[0]
        fm = dit_oracle.attention_module_torch(wm, x, None, angles, H, D, dtype=torch.float64)[0]
        fd = float((dout * (fp - fm)).sum()) / (2 * h)
        assert abs(fd - float((grads[name] * dirw).sum())) < 1e-6, name
