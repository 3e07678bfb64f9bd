"""Pins for the CPU oracle of the DiT block (no GPU): a step-by-step fp64 recomputation with explicit statistics,
central finite differences, and the reference's initialisation property."""
import math

import numpy as np
import pytest
import torch


def make_block_weights(D, Kc, H, lora_dim, seed, zero_last=False):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    hd = D // H
    w = {}
    for pre, kc in (("self_attn.", D), ("cross_attn.", Kc)):
        w[pre + "q_proj.weight"] = r(D, D) / D ** 0.5
        w[pre + "k_proj.weight"] = r(D, kc) / kc ** 0.5
        w[pre + "v_proj.weight"] = r(D, kc) / kc ** 0.5
        w[pre + "output_proj.weight"] = r(D, D) / D ** 0.5
        w[pre + "q_norm.weight"] = 1 + 0.2 * r(hd)
        w[pre + "k_norm.weight"] = 1 + 0.2 * r(hd)
    w["mlp.layer1.weight"] = r(4 * D, D) / D ** 0.5
    w["mlp.layer2.weight"] = r(D, 4 * D) / (4 * D) ** 0.5
    for name in ("self_attn", "cross_attn", "mlp"):
        if lora_dim:
            w[f"adaln_modulation_{name}.1.weight"] = r(lora_dim, D) / D ** 0.5
            w[f"adaln_modulation_{name}.2.weight"] = torch.zeros(3 * D, lora_dim, dtype=torch.float64) if zero_last else r(3 * D, lora_dim) / lora_dim ** 0.5
        else:
            w[f"adaln_modulation_{name}.1.weight"] = torch.zeros(3 * D, D, dtype=torch.float64) if zero_last else r(3 * D, D) / D ** 0.5
    return w


def inputs(B, T, Hh, W, D, Mk, Kc, lora, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    return dict(x=r(B, T, Hh, W, D), emb=r(B, T, D), ctx=r(B, Mk, Kc), lora=(0.3 * r(B, T, 3 * D) if lora else None),
                tx=0.3 * r(B, T, Hh, W, D), temb=0.3 * r(B, T, D), tlora=(0.1 * r(B, T, 3 * D) if lora else None))


@pytest.mark.parametrize("lora_dim", [0, 8])
def test_block_oracle_matches_stepwise_fp64_recomputation(block_oracle, dit_oracle, lora_dim):
    B, T, Hh, W, D, H, Mk, Kc = 2, 2, 2, 3, 32, 2, 5, 24
    w = make_block_weights(D, Kc, H, lora_dim, 1)
    i = inputs(B, T, Hh, W, D, Mk, Kc, bool(lora_dim), 2)
    half = np.random.default_rng(3).standard_normal((T * Hh * W, D // H // 2))
    angles = np.concatenate([half, half], -1)
    out, _ = block_oracle.block_torch(w, i["x"], i["emb"], i["ctx"], angles, H, i["lora"], dtype=torch.float64)

    n64 = lambda t: t.numpy()
    x = n64(i["x"])

    def modulation(name):
        e = n64(i["emb"])
        m = (e / (1 + np.exp(-e))) @ n64(w[f"adaln_modulation_{name}.1.weight"]).T       # SiLU(e) = e * sigmoid(e)
        if lora_dim:
            m = m @ n64(w[f"adaln_modulation_{name}.2.weight"]).T + n64(i["lora"])
        shift, scale, gate = m[..., :D], m[..., D:2 * D], m[..., 2 * D:]
        return [z[:, :, None, None, :] for z in (shift, scale, gate)]

    def ln(t):     # explicit statistics, biased variance, eps inside the root
        mu = t.mean(-1, keepdims=True)
        var = ((t - mu) ** 2).mean(-1, keepdims=True)
        return (t - mu) / np.sqrt(var + 1e-6)

    def attn(prefix, xq, context, ang):
        sub = {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}
        o, _ = dit_oracle.attention_module_torch(sub, torch.from_numpy(xq), None if context is None else torch.from_numpy(context),
                                                 ang, H, D // H, dtype=torch.float64)
        return o.numpy()

    shift, scale, gate = modulation("self_attn")
    n = (ln(x) * (1 + scale) + shift).reshape(B, -1, D)
    x = x + gate * attn("self_attn.", n, None, angles).reshape(x.shape)
    shift, scale, gate = modulation("cross_attn")
    n = (ln(x) * (1 + scale) + shift).reshape(B, -1, D)
    x = x + gate * attn("cross_attn.", n, n64(i["ctx"]), None).reshape(x.shape)
    shift, scale, gate = modulation("mlp")
    n = ln(x) * (1 + scale) + shift
    h = n @ n64(w["mlp.layer1.weight"]).T
    erf = np.vectorize(math.erf)
    x = x + gate * ((0.5 * h * (1 + erf(h / math.sqrt(2)))) @ n64(w["mlp.layer2.weight"]).T)
    np.testing.assert_allclose(out.numpy(), x, atol=1e-10)


@pytest.mark.parametrize("lora_dim", [0, 8])
def test_block_oracle_tangent_matches_central_differences(block_oracle, lora_dim):
    B, T, Hh, W, D, H, Mk, Kc = 1, 2, 2, 2, 32, 2, 4, 16
    w = make_block_weights(D, Kc, H, lora_dim, 4)
    i = inputs(B, T, Hh, W, D, Mk, Kc, bool(lora_dim), 5)
    half = np.random.default_rng(6).standard_normal((T * Hh * W, D // H // 2))
    angles = np.concatenate([half, half], -1)
    _, tout = block_oracle.block_torch(w, i["x"], i["emb"], i["ctx"], angles, H, i["lora"], i["tx"], i["temb"], i["tlora"],
                                       dtype=torch.float64)
    h = 1e-6

    def f(sign):
        lora = None if i["lora"] is None else i["lora"] + sign * h * i["tlora"]
        return block_oracle.block_torch(w, i["x"] + sign * h * i["tx"], i["emb"] + sign * h * i["temb"], i["ctx"], angles, H,
                                        lora, dtype=torch.float64)[0]

    np.testing.assert_allclose(tout.numpy(), ((f(+1) - f(-1)) / (2 * h)).numpy(), atol=2e-7)


def test_block_with_zero_last_modulation_layer_is_the_identity(block_oracle):
    """The reference initialises the last modulation layer to zero (minimal_v4_dit.py:1095-1111): gate = 0, out = x."""
    B, T, Hh, W, D, H, Mk, Kc = 1, 2, 2, 2, 32, 2, 4, 16
    for lora_dim in (0, 8):
        w = make_block_weights(D, Kc, H, lora_dim, 7, zero_last=True)
        i = inputs(B, T, Hh, W, D, Mk, Kc, False, 8)
        lora = torch.zeros(B, T, 3 * D, dtype=torch.float64) if lora_dim else None
        out, tout = block_oracle.block_torch(w, i["x"], i["emb"], i["ctx"], None, H, lora, i["tx"], i["temb"], dtype=torch.float64)
        assert torch.equal(out, i["x"]) and torch.equal(tout, i["tx"])


def test_elementwise_oracles_match_closed_forms(block_oracle):
    """LayerNorm tangent tn = r (tc - n mean(n tc)) and GELU' = Phi + h phi, written out in fp64 numpy, against the
    forward-AD oracles (fp32), plus central differences of the library functions in fp64."""
    g = torch.Generator().manual_seed(31)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    rows, D, rpg = 12, 48, 4
    x, tx = r(rows, D) * 2 + 0.5, r(rows, D)
    sh, sc, tsh, tsc = r(rows // rpg, D), 0.3 * r(rows // rpg, D), r(rows // rpg, D), r(rows // rpg, D)
    y, ty = block_oracle.ln_modulate_torch(x, sh, sc, tx, tsh, tsc, rows_per_group=rpg)
    xn, tn_ = x.numpy(), tx.numpy()
    mu = xn.mean(-1, keepdims=True); xc = xn - mu
    rr = 1 / np.sqrt((xc ** 2).mean(-1, keepdims=True) + 1e-6)
    n = xc * rr
    tc = tn_ - tn_.mean(-1, keepdims=True)
    tn = rr * (tc - n * (n * tc).mean(-1, keepdims=True))
    rep = lambda m: np.repeat(m.numpy(), rpg, axis=0)
    np.testing.assert_allclose(y.numpy(), n * (1 + rep(sc)) + rep(sh), atol=2e-5)
    np.testing.assert_allclose(ty.numpy(), tn * (1 + rep(sc)) + n * rep(tsc) + rep(tsh), atol=2e-5)
    # the LayerNorm tangent against central differences in fp64
    f = lambda z: torch.nn.functional.layer_norm(z, (D,), eps=1e-6).numpy()
    np.testing.assert_allclose(tn, (f(x + 1e-6 * tx) - f(x - 1e-6 * tx)) / 2e-6, atol=1e-7)

    h, th = r(5, 64) * 2, r(5, 64)
    a, ta = block_oracle.gelu_torch(h, th)
    hn = h.numpy()
    erf = np.vectorize(math.erf)
    cdf, pdf = 0.5 * (1 + erf(hn / math.sqrt(2))), np.exp(-0.5 * hn ** 2) / math.sqrt(2 * math.pi)
    np.testing.assert_allclose(a.numpy(), hn * cdf, atol=2e-6)
    np.testing.assert_allclose(ta.numpy(), th.numpy() * (cdf + hn * pdf), atol=2e-6)

    xx, res, gate, txx, tres, tgate = r(rows, D), r(rows, D), r(rows // rpg, D), r(rows, D), r(rows, D), r(rows // rpg, D)
    o, to = block_oracle.gated_residual_torch(xx, res, gate, txx, tres, tgate, rows_per_group=rpg)
    np.testing.assert_allclose(o.numpy(), xx.numpy() + rep(gate) * res.numpy(), atol=2e-6)
    np.testing.assert_allclose(to.numpy(), txx.numpy() + rep(tgate) * res.numpy() + rep(gate) * tres.numpy(), atol=2e-6)


def test_image_branch_is_a_second_attention_summed_before_the_output_projection(block_oracle, dit_oracle):
    """minimal_v4_dit.py:480-483: out_proj(attn(q, k, v) + attn(q, k_img, v_img)).  With zero gates on the other two
    sub-layers the block reduces to x + gate * that, which is rebuilt here from the pinned attention-module oracle by
    linearity of the output projection."""
    B, T, Hh, W, D, H, Mk, Kc, Mi, Ki = 1, 1, 2, 3, 32, 2, 5, 24, 4, 20
    w = make_block_weights(D, Kc, H, 0, 51)
    g = torch.Generator().manual_seed(52)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    w["cross_attn.k_img.weight"], w["cross_attn.v_img.weight"] = r(D, Ki) / Ki ** 0.5, r(D, Ki) / Ki ** 0.5
    w["cross_attn.k_img_norm.weight"] = 1 + 0.2 * r(D // H)
    for name in ("self_attn", "mlp"):                       # gates of the other sub-layers to zero
        w[f"adaln_modulation_{name}.1.weight"][2 * D:] = 0
    i = inputs(B, T, Hh, W, D, Mk, Kc, False, 53)
    img = r(B, Mi, Ki)
    out, _ = block_oracle.block_torch(w, i["x"], i["emb"], (i["ctx"], img), None, H, dtype=torch.float64)

    m = torch.nn.functional.silu(i["emb"]) @ w["adaln_modulation_cross_attn.1.weight"].T
    shift, scale, gate = (c[:, :, None, None, :] for c in m.chunk(3, dim=-1))
    n = (torch.nn.functional.layer_norm(i["x"], (D,), eps=1e-6) * (1 + scale) + shift).reshape(B, -1, D)
    text = {k[len("cross_attn."):]: v for k, v in w.items() if k.startswith("cross_attn.") and "img" not in k}
    image = dict(text)
    image["k_proj.weight"], image["v_proj.weight"], image["k_norm.weight"] = (w["cross_attn.k_img.weight"], w["cross_attn.v_img.weight"],
                                                                              w["cross_attn.k_img_norm.weight"])
    a1, _ = dit_oracle.attention_module_torch(text, n, i["ctx"], None, H, D // H, dtype=torch.float64)
    a2, _ = dit_oracle.attention_module_torch(image, n, img, None, H, D // H, dtype=torch.float64)
    want = i["x"] + gate * (a1 + a2).reshape(i["x"].shape)
    np.testing.assert_allclose(out.numpy(), want.numpy(), atol=1e-10)
