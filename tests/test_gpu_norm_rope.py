"""GPU parity of the fused RMSNorm + rotary (+ tangent) kernel, called through the C ABI, against the CPU oracle.

Oracle: numpy fp64 closed form, pinned to torch's rms_norm under forward AD (tests/test_oracle_norm_rope.py).
Two bars, both written here:
  * against the unrounded fp64 result: max-abs <= 2e-2 * max(1, max|want|) and relative-L2 <= 5e-3 (the path's
    16-bit tolerance; the result carries two 16-bit roundings, RMSNorm's output and the final store);
  * against the oracle with the same rounding point (RMSNorm's output rounded to the 16-bit type): every element
    within the bound that 16-bit rounding alone allows, and at least 97% of the elements bit-equal to the correctly
    rounded oracle value.
"""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ABS, REL_L2 = 2e-2, 5e-3
HALF_ULP = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}   # relative bound of one rounding to the type
HALF = {torch.bfloat16: "bf16", torch.float16: "fp16"}


def check(name, got_t, want, want_rounded, n_rounded, dtype):
    """want: fp64 result without intermediate rounding; want_rounded: fp64 result from the 16-bit-rounded
    normalised tensor n_rounded (the kernel's rounding point)."""
    got = got_t.float().cpu().double().numpy()
    ma = float(np.abs(got - want).max())
    rl = float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30))
    lim = MAX_ABS * max(1.0, float(np.abs(want).max()))
    # second bar.  The final store rounds once (<= HALF_ULP * |y|).  The kernel forms n in fp32, the oracle in fp64:
    # where the two land on different sides of a rounding boundary n moves by one unit in the last place
    # (<= 2 * HALF_ULP * |n|), and that moves y by at most the same amount for each of the two n that enter it.
    D = n_rounded.shape[-1]
    partner = np.concatenate([n_rounded[..., D // 2:], n_rounded[..., : D // 2]], axis=-1)
    U = HALF_ULP[dtype]
    tol = U * np.abs(want_rounded) + 2 * U * (np.abs(n_rounded) + np.abs(partner)) + 1e-7
    worst = float((np.abs(got - want_rounded) / tol).max())
    # and nearly every element is the correctly rounded value of the oracle's
    exact = torch.from_numpy(want_rounded).to(dtype).double().numpy() == got
    frac = float(exact.mean())
    print(f"  {name}: max_abs={ma:.3e} (limit {lim:.3e}) rel_l2={rl:.3e} worst/tol={worst:.2f} bit-equal={frac:.4f}", flush=True)
    assert math.isfinite(ma) and ma <= lim, f"{name}: max-abs {ma} > {lim}"
    assert rl <= REL_L2, f"{name}: rel-L2 {rl} > {REL_L2}"
    assert worst <= 1.0, f"{name}: {worst} x the rounding bound from the oracle with the same rounding point"
    assert frac >= 0.97, f"{name}: only {frac} of the elements equal the rounded oracle value"


def check_all(nr_oracle, y, ty, x, w, a, tx, dtype, suffix=""):
    want, twant = nr_oracle.norm_rope_closed_form(x, w, a, tx, eps=1e-6)
    wr, twr = nr_oracle.norm_rope_closed_form(x, w, a, tx, eps=1e-6, half=HALF[dtype])
    n, tn = nr_oracle.norm_rope_closed_form(x, w, None, tx, eps=1e-6, half=HALF[dtype])
    check("y" + suffix, y, want, wr, n, dtype)
    if tx is not None:
        check("ty" + suffix, ty, twant, twr, tn, dtype)
    else:
        assert ty is None


def run_case(pkg, nr_oracle, gpu, B, S, H, D, dtype=torch.bfloat16, rope=True, tangent=True, weight=True, seed=0,
             out_layout="bshd", x_std=1.0, strided=False, angle_scale=None):
    g = torch.Generator().manual_seed(seed)
    print(f"norm_rope case B={B} S={S} H={H} D={D} {dtype} rope={rope} tangent={tangent} weight={weight} "
          f"layout={out_layout} strided={strided} seed={seed}", flush=True)
    if strided:
        # q as a slice of a fused [B, S, 3, H, D] projection output
        full = (torch.randn(B, S, 3, H, D, generator=g) * x_std).to(dtype)
        tfull = (torch.randn(B, S, 3, H, D, generator=g) * 0.3).to(dtype)
        x, tx = full[:, :, 1], tfull[:, :, 1]
        xd, txd = full.to(gpu)[:, :, 1], tfull.to(gpu)[:, :, 1]
    else:
        x = (torch.randn(B, S, H, D, generator=g) * x_std).to(dtype)
        tx = (torch.randn(B, S, H, D, generator=g) * 0.3).to(dtype)
        xd, txd = x.to(gpu), tx.to(gpu)
    w = (1.0 + 0.2 * torch.randn(D, generator=g)) if weight else None
    if rope:
        if angle_scale is None:
            a = torch.from_numpy(nr_oracle.rope_angles_3d(1, 1, S, D))          # positions 0..S-1 along w
        else:
            half = torch.randn(S, D // 2, generator=g) * angle_scale
            a = torch.cat([half, half], dim=-1).float()
        rope_emb = a.reshape(S, 1, 1, D)
    else:
        a = rope_emb = None
    y, ty = pkg.norm_rope(xd, None if w is None else w.to(gpu), None if rope_emb is None else rope_emb.to(gpu),
                          txd if tangent else None, eps=1e-6, out_layout=out_layout)
    torch.cuda.synchronize()
    assert y.shape == (B, S, H, D) and y.dtype == dtype
    if out_layout == "bhsd":
        assert y.transpose(1, 2).is_contiguous()
    wn = None if w is None else w.float().numpy()
    an = None if a is None else a.numpy()
    check_all(nr_oracle, y, ty, x.float().numpy(), wn, an, tx.float().numpy() if tangent else None, dtype)
    return y, ty


def test_smallest(pkg, nr_oracle, gpu):
    run_case(pkg, nr_oracle, gpu, 1, 1, 1, 128)


@pytest.mark.parametrize("D", [16, 32, 64, 128, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_head_dims_and_dtypes(pkg, nr_oracle, gpu, D, dtype):
    run_case(pkg, nr_oracle, gpu, 2, 37, 3, D, dtype=dtype, seed=D)


@pytest.mark.parametrize("H", [1, 2, 3, 4, 5, 7, 8, 16])
def test_head_counts_around_the_group_of_four(pkg, nr_oracle, gpu, H):
    run_case(pkg, nr_oracle, gpu, 1, 19, H, 128, seed=H)
    run_case(pkg, nr_oracle, gpu, 2, 5, H, 32, seed=100 + H)


@pytest.mark.parametrize("rope,tangent,weight", [(True, False, True), (False, True, True), (False, False, False),
                                                 (True, True, False)])
def test_optional_operands(pkg, nr_oracle, gpu, rope, tangent, weight):
    run_case(pkg, nr_oracle, gpu, 1, 50, 4, 128, rope=rope, tangent=tangent, weight=weight, seed=7)


@pytest.mark.parametrize("S", [1, 15, 16, 17, 255, 1000])
def test_ragged_row_counts(pkg, nr_oracle, gpu, S):
    run_case(pkg, nr_oracle, gpu, 1, S, 5, 64, seed=S)


def test_heads_first_output_and_strided_input(pkg, nr_oracle, gpu):
    a, ta = run_case(pkg, nr_oracle, gpu, 2, 33, 6, 128, out_layout="bshd", seed=3)
    b, tb = run_case(pkg, nr_oracle, gpu, 2, 33, 6, 128, out_layout="bhsd", seed=3)
    assert torch.equal(a, b) and torch.equal(ta, tb)
    c, tc = run_case(pkg, nr_oracle, gpu, 2, 33, 6, 128, strided=True, seed=4)
    # the same slice made contiguous gives the same bits
    d, td = run_case(pkg, nr_oracle, gpu, 2, 33, 6, 128, strided=True, seed=4, out_layout="bhsd")
    assert torch.equal(c, d) and torch.equal(tc, td)


def test_large_angles_and_scaled_inputs(pkg, nr_oracle, gpu):
    # angles of a few hundred radians (late positions at frequency 1) and inputs far from unit scale
    run_case(pkg, nr_oracle, gpu, 1, 64, 4, 128, angle_scale=300.0, seed=11)
    run_case(pkg, nr_oracle, gpu, 1, 64, 4, 128, x_std=40.0, seed=12)
    run_case(pkg, nr_oracle, gpu, 1, 64, 4, 128, x_std=1e-2, seed=13)


def test_video_positions(pkg, nr_oracle, gpu):
    """Angles of a (T, H, W) = (3, 6, 10) token grid, as the DiT's positional embedding lays them out."""
    T, Hh, W, D, H = 3, 6, 10, 128, 4
    S = T * Hh * W
    g = torch.Generator().manual_seed(21)
    x = torch.randn(1, S, H, D, generator=g).bfloat16()
    tx = (torch.randn(1, S, H, D, generator=g) * 0.3).bfloat16()
    a = nr_oracle.rope_angles_3d(T, Hh, W, D)
    y, ty = pkg.norm_rope(x.to(gpu), None, torch.from_numpy(a).reshape(S, 1, 1, D).to(gpu), tx.to(gpu))
    check_all(nr_oracle, y, ty, x.float().numpy(), None, a, tx.float().numpy(), torch.bfloat16)


def test_full_size_invariants(pkg, nr_oracle, gpu):
    """At the size of one DiT self-attention (S = 84480 tokens, 16 heads of 128): properties that need no CPU pass
    over the whole tensor, plus the oracle on a sample of rows."""
    B, S, H, D = 1, 84480, 16, 128
    g = torch.Generator(device=gpu).manual_seed(5)
    x = torch.randn(B, S, H, D, generator=g, device=gpu).bfloat16()
    tx = (torch.randn(B, S, H, D, generator=g, device=gpu) * 0.3).bfloat16()
    a = torch.from_numpy(nr_oracle.rope_angles_3d(24, 44, 80, D)).to(gpu)
    y, ty = pkg.norm_rope(x, None, a, tx)
    n, tn = pkg.norm_rope(x, None, None, tx)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all() and torch.isfinite(ty.float()).all()
    # the rotation keeps the length of every (j, j + D/2) pair, up to the final 16-bit rounding
    pl = lambda t: t.float()[..., : D // 2] ** 2 + t.float()[..., D // 2 :] ** 2
    pl_err, pl_max = float((pl(y) - pl(n)).abs().max()), float(pl(n).max())
    assert pl_err <= 4 * 2.0 ** -8 * pl_max, (pl_err, pl_max)
    # unit weight: every normalised row has mean square 1 up to 16-bit rounding (each element moves by at most
    # 2^-8 of itself, its square by at most 2^-7 of itself, and so does the mean of the squares)
    ms_err = float(((n.float() ** 2).mean(-1) - 1).abs().max())
    assert ms_err <= 2.0 ** -7 + 1e-4, ms_err
    # position 0 has angle 0: the rotation is the identity there
    assert torch.equal(y[:, 0], n[:, 0]) and torch.equal(ty[:, 0], tn[:, 0])
    # tangent along x itself vanishes (scale invariance), up to eps and rounding
    _, tself = pkg.norm_rope(x, None, a, x)
    tself_max = float(tself.float().abs().max())
    assert tself_max <= 1e-4, tself_max
    # the oracle on a sample of positions
    idx = torch.tensor([0, 1, 79, 80, 3519, 3520, 42239, 84479], device=gpu)
    xs, txs, as_ = x[:, idx].cpu().float().numpy(), tx[:, idx].cpu().float().numpy(), a[idx].cpu().numpy()
    check_all(nr_oracle, y[:, idx], ty[:, idx], xs, None, as_, txs, torch.bfloat16, suffix="[sample]")


def test_feeds_the_attention_kernel_without_a_transpose(pkg, oracle, nr_oracle, gpu):
    """norm_rope(..., out_layout="bhsd") -> attention_jvp, against the oracles chained the same way."""
    B, S, H, D = 1, 200, 2, 128
    g = torch.Generator().manual_seed(9)
    mk = lambda std: (torch.randn(B, S, H, D, generator=g) * std).bfloat16()
    xq, xk, v, tq, tk, tv = mk(1), mk(1), mk(1), mk(0.3), mk(0.3), mk(0.3)
    a = torch.from_numpy(nr_oracle.rope_angles_3d(1, 10, 20, D))
    ad = a.to(gpu)
    q, dq = pkg.norm_rope(xq.to(gpu), None, ad, tq.to(gpu), out_layout="bhsd")
    k, dk = pkg.norm_rope(xk.to(gpu), None, ad, tk.to(gpu), out_layout="bhsd")
    bh = lambda t: t.transpose(1, 2)      # [B, H, S, D] views, already contiguous in that order for q, k
    o, to = pkg.attention_jvp(bh(q), bh(k), bh(v.to(gpu)), bh(dq), bh(dk), bh(tv.to(gpu)))
    torch.cuda.synchronize()
    f = lambda t: t.float().numpy()
    qr, dqr = nr_oracle.norm_rope_closed_form(f(xq), None, a.numpy(), f(tq))
    kr, dkr = nr_oracle.norm_rope_closed_form(f(xk), None, a.numpy(), f(tk))
    t = lambda z: np.ascontiguousarray(np.swapaxes(z, 1, 2))
    o_ref, to_ref, _ = oracle.closed_form(t(qr), t(kr), t(f(v)), t(dqr), t(dkr), t(f(tv)))
    for name, got, want in (("o", o, o_ref), ("to", to, to_ref)):
        ma, rl = oracle.error_metrics(got.float().cpu(), want)
        print(f"  {name}: max_abs={ma:.3e} rel_l2={rl:.3e}", flush=True)
        assert ma <= 2e-2 and rl <= 1e-2


# ---------------------------------------------------------------------------------------------- reverse mode
def check_grad(name, got, want, max_abs=MAX_ABS, rel_l2=REL_L2):
    got = got.float().cpu().double().numpy()
    ma = float(np.abs(got - want).max())
    rl = float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30))
    lim = max_abs * max(1.0, float(np.abs(want).max()))
    print(f"  {name}: max_abs={ma:.3e} (limit {lim:.3e}) rel_l2={rl:.3e}", flush=True)
    assert math.isfinite(ma) and ma <= lim, f"{name}: max-abs {ma} > {lim}"
    assert rl <= rel_l2, f"{name}: rel-L2 {rl} > {rel_l2}"


def run_bwd_case(pkg, nr_oracle, gpu, B, S, H, D, dtype=torch.bfloat16, rope=True, weight=True, seed=0, dy_layout="bshd",
                 need_dweight=True):
    print(f"norm_rope_bwd case B={B} S={S} H={H} D={D} {dtype} rope={rope} weight={weight} dy_layout={dy_layout} seed={seed}", flush=True)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, S, H, D, generator=g).to(dtype)
    dy = torch.randn(B, S, H, D, generator=g).to(dtype)
    w = (1.0 + 0.2 * torch.randn(D, generator=g)) if weight else None
    a = torch.from_numpy(nr_oracle.rope_angles_3d(1, 1, S, D)) if rope else None
    dyd = dy.to(gpu)
    if dy_layout == "bhsd":     # the gradient as the attention backward hands it over: heads-first memory
        dyd = dyd.transpose(1, 2).contiguous().transpose(1, 2)
    dx, dw = pkg.norm_rope_bwd(x.to(gpu), None if w is None else w.to(gpu), None if a is None else a.to(gpu), dyd,
                               need_dweight=need_dweight)
    torch.cuda.synchronize()
    assert dx.shape == x.shape and dx.dtype == dtype and dx.is_contiguous()
    want_dx, want_dw = nr_oracle.norm_rope_grads_closed_form(x.float().numpy(), None if w is None else w.numpy(),
                                                             None if a is None else a.numpy(), dy.float().numpy())
    check_grad("dx", dx, want_dx)
    if need_dweight:
        assert dw.dtype == torch.float32 and dw.shape == (D,)
        check_grad("dweight", dw, want_dw, rel_l2=2e-3)     # fp32 sums of products of 16-bit inputs
    else:
        assert dw is None
    return dx, dw


@pytest.mark.parametrize("D", [16, 32, 64, 128, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_bwd_head_dims_and_dtypes(pkg, nr_oracle, gpu, D, dtype):
    run_bwd_case(pkg, nr_oracle, gpu, 2, 37, 3, D, dtype=dtype, seed=D)


@pytest.mark.parametrize("H", [1, 3, 4, 5, 16])
@pytest.mark.parametrize("S", [1, 17, 300])
def test_bwd_ragged_sizes(pkg, nr_oracle, gpu, H, S):
    run_bwd_case(pkg, nr_oracle, gpu, 1, S, H, 128, seed=H * 1000 + S)


@pytest.mark.parametrize("rope,weight", [(False, True), (True, False), (False, False)])
def test_bwd_optional_operands(pkg, nr_oracle, gpu, rope, weight):
    run_bwd_case(pkg, nr_oracle, gpu, 1, 50, 4, 64, rope=rope, weight=weight, seed=5)


def test_bwd_strided_gradient_no_dweight_and_determinism(pkg, nr_oracle, gpu):
    a, wa = run_bwd_case(pkg, nr_oracle, gpu, 2, 130, 6, 128, dy_layout="bhsd", seed=6)
    b, wb = run_bwd_case(pkg, nr_oracle, gpu, 2, 130, 6, 128, dy_layout="bshd", seed=6)
    assert torch.equal(a, b) and torch.equal(wa, wb)            # same values through either gradient layout, bit for bit
    c, _ = run_bwd_case(pkg, nr_oracle, gpu, 2, 130, 6, 128, seed=6, need_dweight=False)
    assert torch.equal(a, c)


def test_bwd_many_blocks_dweight_reduction(pkg, nr_oracle, gpu):
    """Enough rows for thousands of partial-sum rows: the two-stage dweight reduction against the oracle."""
    run_bwd_case(pkg, nr_oracle, gpu, 1, 20000, 16, 128, seed=8)


def test_autograd_through_norm_rope_matches_the_raw_op(pkg, nr_oracle, gpu):
    torch.manual_seed(0)
    m = pkg.Attention(256, None, n_heads=2, head_dim=128).to(device=gpu, dtype=torch.bfloat16)
    x = torch.randn(1, 40, 2, 128, device=gpu, dtype=torch.bfloat16, requires_grad=True)
    a = torch.from_numpy(nr_oracle.rope_angles_3d(1, 1, 40, 128)).to(gpu)
    y, _ = m._norm_rope(x, m.q_norm, a)
    dy = torch.randn_like(y)
    y.backward(dy)
    dx, dw = pkg.norm_rope_bwd(x.detach(), m.q_norm.weight.detach(), a, dy)
    assert torch.equal(x.grad, dx) and torch.equal(m.q_norm.weight.grad, dw.to(torch.bfloat16))


def test_more_than_2_31_elements(pkg, nr_oracle, gpu):
    """Offsets beyond 32 bits: x of 2.2e9 elements (4.5 GB); the last rows and a sample in between against the oracle."""
    B, S, H, D = 1, 131072, 132, 128
    assert B * S * H * D > 2 ** 31
    x = torch.empty(B, S, H, D, device=gpu, dtype=torch.bfloat16)
    g = torch.Generator(device=gpu).manual_seed(3)
    for i in range(0, S, 16384):            # fill in slabs: no fp32 temporary of the whole tensor
        x[:, i:i + 16384] = torch.randn(B, 16384, H, D, generator=g, device=gpu).bfloat16()
    half = torch.randn(S, D // 2, generator=g, device=gpu)
    a = torch.cat([half, half], dim=-1)
    w = (1.0 + 0.2 * torch.randn(D, generator=g, device=gpu)).float()
    y, _ = pkg.norm_rope(x, w, a)
    torch.cuda.synchronize()
    idx = torch.tensor([0, 1, 65535, 65536, 127073, 131070, 131071], device=gpu)     # rows on both sides of 2^31 elements
    xs, as_ = x[:, idx].cpu().float().numpy(), a[idx].cpu().numpy()
    want, _ = nr_oracle.norm_rope_closed_form(xs, w.cpu().numpy(), as_)
    wr, _ = nr_oracle.norm_rope_closed_form(xs, w.cpu().numpy(), as_, half="bf16")
    n, _ = nr_oracle.norm_rope_closed_form(xs, w.cpu().numpy(), None, half="bf16")
    check("y[sample]", y[:, idx], want, wr, n, torch.bfloat16)
    # every row was written: unit mean square over the weight-free part cannot be checked with a weight, so check finiteness
    # and that no row was left at the allocator's garbage by comparing two far-apart slabs' statistics
    assert torch.isfinite(y[:, -4096:].float()).all() and float(y[:, -4096:].float().abs().mean()) > 0.5
    del y
    dx, dw = pkg.norm_rope_bwd(x, w, a, x)          # reverse mode on the same size (dy = x)
    torch.cuda.synchronize()
    want_dx, _ = nr_oracle.norm_rope_grads_closed_form(xs, w.cpu().numpy(), as_, xs)
    check_grad("dx[sample]", dx[:, idx], want_dx)
    assert torch.isfinite(dw).all()
