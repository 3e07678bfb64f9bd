"""GPU parity of the fused elementwise steps of the DiT block (LayerNorm + modulation, gated residual, GELU; each with
its tangent), called through the C ABI, against the CPU oracle (library layer_norm / gelu under torch.func.jvp, fp32,
pinned in tests/test_oracle_dit_block.py).

Tolerance: one 16-bit rounding of an fp32 result, with a quarter of slack for the fp32 arithmetic itself:
|got - want| <= 1.25 * 2^-8 |want| + 1e-3 elementwise for bf16 (1.25 * 2^-11 |want| + 2e-4 for fp16; the absolute term
covers cancellation near zero), and
relative-L2 <= 3e-3 (bf16) / 5e-4 (fp16).
"""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

REL = {torch.bfloat16: (1.25 * 2.0 ** -8, 1e-3, 3e-3), torch.float16: (1.25 * 2.0 ** -11, 2e-4, 5e-4)}


def check(name, got, want, dtype):
    got, want = got.float().cpu().double(), want.double()
    rel, ab, l2 = REL[dtype]
    err = (got - want).abs()
    worst = float((err / (rel * want.abs() + ab)).max())
    rl = float((got - want).norm() / want.norm().clamp_min(1e-30))
    print(f"  {name}: worst/tol={worst:.2f} rel_l2={rl:.3e}", flush=True)
    assert math.isfinite(worst) and worst <= 1.0, f"{name}: {worst} x the elementwise bound"
    assert rl <= l2, f"{name}: rel-L2 {rl} > {l2}"


def rnd(g, dtype, *shape, std=1.0, mean=0.0):
    return (torch.randn(*shape, generator=g) * std + mean).to(dtype)


@pytest.mark.parametrize("D", [8, 64, 256, 520, 2048, 5120, 8192])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_ln_modulate_widths(pkg, block_oracle, gpu, D, dtype):
    g = torch.Generator().manual_seed(D)
    rows, rpg = 24, 4
    x, tx = rnd(g, dtype, rows, D, std=2.0, mean=0.5), rnd(g, dtype, rows, D, std=0.5)
    sh, sc, tsh, tsc = (rnd(g, dtype, rows // rpg, D, std=s) for s in (1.0, 0.3, 0.3, 0.1))
    print(f"ln_modulate D={D} {dtype}", flush=True)
    d = lambda t: t.to(gpu)
    y, ty = pkg.ln_modulate(d(x), d(sh), d(sc), d(tx), d(tsh), d(tsc))
    want, twant = block_oracle.ln_modulate_torch(x, sh, sc, tx, tsh, tsc, rows_per_group=rpg)
    check("y", y, want, dtype)
    check("ty", ty, twant, dtype)
    # values only, and a tangent with a modulation that does not move
    y2, none = pkg.ln_modulate(d(x), d(sh), d(sc))
    assert none is None
    check("y (values only)", y2, want, dtype)      # another instantiation of the kernel: same bar, not the same bits
    y3, ty3 = pkg.ln_modulate(d(x), d(sh), d(sc), d(tx))
    _, twant3 = block_oracle.ln_modulate_torch(x, sh, sc, tx, rows_per_group=rpg)
    check("y (fixed modulation)", y3, want, dtype)
    check("ty (fixed modulation)", ty3, twant3, dtype)


def test_ln_modulate_video_shape_and_stacked_output(pkg, block_oracle, gpu):
    g = torch.Generator().manual_seed(1)
    B, T, Hh, W, D = 2, 3, 4, 5, 256
    x, tx = rnd(g, torch.bfloat16, B, T, Hh, W, D), rnd(g, torch.bfloat16, B, T, Hh, W, D)
    sh, sc = rnd(g, torch.bfloat16, B * T, D), rnd(g, torch.bfloat16, B * T, D, std=0.3)
    y, ty = pkg.ops.stacked_pair(x.shape, x.dtype, gpu)
    pkg.ln_modulate(x.to(gpu), sh.to(gpu), sc.to(gpu), tx.to(gpu), out=y, tout=ty)
    both = pkg.ops.as_stacked(y.reshape(B, -1, D), ty.reshape(B, -1, D))
    assert both is not None and both.shape == (2 * B, T * Hh * W, D) and both.data_ptr() == y.data_ptr()
    assert pkg.ops.as_stacked(y.clone(), ty.clone()) is None
    want, twant = block_oracle.ln_modulate_torch(x, sh, sc, tx, rows_per_group=Hh * W)
    check("y", y, want, torch.bfloat16)
    check("ty", ty, twant, torch.bfloat16)


def test_ln_modulate_large_mean(pkg, block_oracle, gpu):
    """Rows whose mean is far larger than their spread: the variance is taken around the mean, not from raw moments."""
    g = torch.Generator().manual_seed(2)
    x = rnd(g, torch.bfloat16, 8, 2048, std=0.5, mean=60.0)
    sh, sc = torch.zeros(1, 2048).bfloat16(), torch.zeros(1, 2048).bfloat16()
    y, _ = pkg.ln_modulate(x.to(gpu), sh.to(gpu), sc.to(gpu))
    want, _ = block_oracle.ln_modulate_torch(x, sh, sc, rows_per_group=8)
    check("y", y, want, torch.bfloat16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,D,rpg", [(1, 8, 1), (30, 264, 5), (64, 2048, 16)])
def test_gated_residual(pkg, block_oracle, gpu, dtype, rows, D, rpg):
    g = torch.Generator().manual_seed(rows + D)
    x, res, tx, tres = (rnd(g, dtype, rows, D) for _ in range(4))
    gate, tgate = rnd(g, dtype, rows // rpg, D), rnd(g, dtype, rows // rpg, D, std=0.3)
    d = lambda t: t.to(gpu)
    out, tout = pkg.gated_residual(d(x), d(res), d(gate), d(tx), d(tres), d(tgate))
    want, twant = block_oracle.gated_residual_torch(x, res, gate, tx, tres, tgate, rows_per_group=rpg)
    check("out", out, want, dtype)
    check("tout", tout, twant, dtype)
    o2, none = pkg.gated_residual(d(x), d(res), d(gate))
    assert none is None
    check("out (values only)", o2, want, dtype)
    xd, txd = d(x), d(tx)
    o3, t3 = pkg.gated_residual(xd, d(res), d(gate), txd, d(tres), None, inplace=True)
    assert o3.data_ptr() == xd.data_ptr() and t3.data_ptr() == txd.data_ptr() and torch.equal(o3, out)
    _, twant3 = block_oracle.gated_residual_torch(x, res, gate, tx, tres, None, rows_per_group=rpg)
    check("tout (fixed gate, in place)", t3, twant3, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [8, 1000, 1 << 20])
def test_gelu(pkg, block_oracle, gpu, dtype, n):
    g = torch.Generator().manual_seed(n)
    h, th = rnd(g, dtype, n, std=2.5), rnd(g, dtype, n)
    a, ta = pkg.gelu(h.to(gpu), th.to(gpu))
    want, twant = block_oracle.gelu_torch(h, th)
    check("a", a, want, dtype)
    check("ta", ta, twant, dtype)
    a2, none = pkg.gelu(h.to(gpu))
    assert none is None
    check("a (values only)", a2, want, dtype)
    hd, thd = h.to(gpu), th.to(gpu)
    a3, ta3 = pkg.gelu(hd, thd, inplace=True)
    assert a3.data_ptr() == hd.data_ptr() and torch.equal(a3, a) and torch.equal(ta3, ta)


def test_gelu_tails(pkg, block_oracle, gpu):
    h = torch.tensor([-40.0, -12.0, -6.0, -1e-3, 0.0, 1e-3, 6.0, 12.0], dtype=torch.bfloat16)
    a, ta = pkg.gelu(h.to(gpu), torch.ones_like(h).to(gpu))
    want, twant = block_oracle.gelu_torch(h, torch.ones_like(h))
    check("a", a, want, torch.bfloat16)
    check("ta", ta, twant, torch.bfloat16)
    assert torch.isfinite(a.float()).all() and torch.isfinite(ta.float()).all()


def test_more_than_2_31_elements(pkg, block_oracle, gpu):
    """Offsets beyond 32 bits in the three elementwise kernels: 2.4e9-element tensors, checked at both ends."""
    rows, D, rpg = 1179648, 2048, 4096
    assert rows * D > 2 ** 31
    g = torch.Generator(device=gpu).manual_seed(4)
    x = torch.empty(rows, D, device=gpu, dtype=torch.bfloat16)
    for i in range(0, rows, 131072):
        x[i:i + 131072] = torch.randn(131072, D, generator=g, device=gpu).bfloat16()
    mod = torch.randn(3, rows // rpg, D, generator=g, device=gpu).bfloat16()
    ends = torch.cat([torch.arange(0, 8), torch.arange(rows - 8, rows)]).to(gpu)
    grp = (ends // rpg)
    y, _ = pkg.ln_modulate(x, mod[0], mod[1])
    want, _ = block_oracle.ln_modulate_torch(x[ends].cpu(), mod[0][grp].cpu(), mod[1][grp].cpu())
    check("ln_modulate ends", y[ends], want, torch.bfloat16)
    out, _ = pkg.gated_residual(x, y, mod[2])
    want, _ = block_oracle.gated_residual_torch(x[ends].cpu(), y[ends].cpu(), mod[2][grp].cpu())
    check("gated_residual ends", out[ends], want, torch.bfloat16)
    del out
    a, _ = pkg.gelu(x)
    want, _ = block_oracle.gelu_torch(x[ends].cpu())
    check("gelu ends", a[ends], want, torch.bfloat16)
