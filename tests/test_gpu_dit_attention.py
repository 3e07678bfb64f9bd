"""GPU parity of the DiT Attention module (backend "hip": library GEMMs + the fused RMSNorm/RoPE kernel + the attention
kernels, all through the C ABI) and of its forward-mode tangent, against the CPU oracle of the module
(torch fp32 under torch.func.jvp, pinned in tests/test_oracle_dit_attention.py) on the same 16-bit weights and inputs.

Tolerance: the module chains four 16-bit stages (projection, normalised q/k, attention output, output projection), each
rounding to 2^-9 relative (bf16); outputs are compared with relative-L2 <= 1e-2 and max-abs <= 3e-2 * max(1, max|want|).
"""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

REL_L2, MAX_ABS = 1e-2, 3e-2


def check(oracle, name, got, want):
    ma, rl = oracle.error_metrics(got.float().cpu(), want)
    lim = MAX_ABS * max(1.0, float(want.abs().max()))
    print(f"  {name}: max_abs={ma:.3e} (limit {lim:.3e}) rel_l2={rl:.3e}", flush=True)
    assert math.isfinite(ma) and ma <= lim, f"{name}: max-abs {ma} > {lim}"
    assert rl <= REL_L2, f"{name}: rel-L2 {rl} > {REL_L2}"


def build(pkg, gpu, K, Kc, H, D, dtype, seed):
    torch.manual_seed(seed)
    m = pkg.Attention(K, Kc, n_heads=H, head_dim=D)
    m.init_weights()
    with torch.no_grad():
        m.q_norm.weight.add_(0.2 * torch.randn(D))
        m.k_norm.weight.add_(0.2 * torch.randn(D))
    return m.to(device=gpu, dtype=dtype).eval()


def run(pkg, oracle, nr_oracle, dit_oracle, gpu, B, Mq, K, H, D, Mk=None, Kc=None, dtype=torch.bfloat16, seed=0,
        moving_context=False, rope=True):
    cross = Kc is not None
    print(f"module case B={B} Mq={Mq} K={K} H={H} D={D} Mk={Mk} Kc={Kc} {dtype} moving_context={moving_context} seed={seed}", flush=True)
    m = build(pkg, gpu, K, Kc, H, D, dtype, seed)
    g = torch.Generator().manual_seed(seed + 1)
    x = torch.randn(B, Mq, K, generator=g).to(dtype)
    tx = (torch.randn(B, Mq, K, generator=g) * 0.3).to(dtype)
    context = torch.randn(B, Mk, Kc, generator=g).to(dtype) if cross else None
    tcontext = (torch.randn(B, Mk, Kc, generator=g) * 0.3).to(dtype) if (cross and moving_context) else None
    angles = torch.from_numpy(nr_oracle.rope_angles_3d(1, 1, Mq, D)) if rope else None
    rope_emb = None if angles is None else angles.reshape(Mq, 1, 1, D).to(gpu)
    d = lambda t: None if t is None else t.to(gpu)
    with torch.no_grad():
        out = m(d(x), d(context), rope_emb=rope_emb)
    out2, tout = m.forward_jvp(d(x), d(tx), d(context), d(tcontext), rope_emb=rope_emb)
    torch.cuda.synchronize()
    assert out.shape == x.shape and out.dtype == dtype and tout.shape == x.shape
    w = {k: v for k, v in m.state_dict().items()}
    want, twant = dit_oracle.attention_module_torch(w, x, context, None if angles is None else angles.numpy(), H, D, tx, tcontext)
    check(oracle, "out", out, want)
    check(oracle, "out (jvp call)", out2, want)
    check(oracle, "tout", tout, twant)


def test_self_attention_small(pkg, oracle, nr_oracle, dit_oracle, gpu):
    run(pkg, oracle, nr_oracle, dit_oracle, gpu, B=2, Mq=100, K=256, H=4, D=64)


@pytest.mark.parametrize("D,H", [(128, 2), (64, 3), (32, 4)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_self_attention_head_dims(pkg, oracle, nr_oracle, dit_oracle, gpu, D, H, dtype):
    run(pkg, oracle, nr_oracle, dit_oracle, gpu, B=1, Mq=333, K=H * D, H=H, D=D, dtype=dtype, seed=D)


def test_self_attention_without_rope(pkg, oracle, nr_oracle, dit_oracle, gpu):
    run(pkg, oracle, nr_oracle, dit_oracle, gpu, B=1, Mq=77, K=128, H=2, D=64, rope=False, seed=3)


@pytest.mark.parametrize("moving_context", [False, True])
def test_cross_attention(pkg, oracle, nr_oracle, dit_oracle, gpu, moving_context):
    # text cross-attention of the DiT: context of another width, no rotation, tangent on x only (or on both)
    run(pkg, oracle, nr_oracle, dit_oracle, gpu, B=2, Mq=200, K=256, H=2, D=128, Mk=48, Kc=96, moving_context=moving_context, seed=5)


def test_dit_block_shape_reduced_length(pkg, oracle, nr_oracle, dit_oracle, gpu):
    """The 2B DiT's self-attention (K = 2048, 16 heads of 128) at a length the CPU oracle finishes in seconds."""
    run(pkg, oracle, nr_oracle, dit_oracle, gpu, B=1, Mq=1536, K=2048, H=16, D=128, seed=9)


def test_video_shaped_input_and_state_dict_round_trip(pkg, oracle, nr_oracle, dit_oracle, gpu):
    B, T, Hh, W, K, H, D = 1, 2, 4, 6, 128, 2, 64
    m = build(pkg, gpu, K, None, H, D, torch.bfloat16, 11)
    m2 = pkg.Attention(K, None, n_heads=H, head_dim=D).to(device=gpu, dtype=torch.bfloat16).eval()
    m2.load_state_dict(m.state_dict())
    g = torch.Generator().manual_seed(12)
    x = torch.randn(B, T, Hh, W, K, generator=g).bfloat16().to(gpu)
    a = torch.from_numpy(nr_oracle.rope_angles_3d(T, Hh, W, D)).to(gpu)
    with torch.no_grad():
        o1, o2 = m(x, rope_emb=a.reshape(-1, 1, 1, D)), m2(x, rope_emb=a.reshape(-1, 1, 1, D))
    assert o1.shape == x.shape and torch.equal(o1, o2)
    want, _ = dit_oracle.attention_module_torch(m.state_dict(), x.reshape(B, -1, K), None, a.cpu().numpy(), H, D)
    check(oracle, "out", o1.reshape(B, -1, K), want)


@pytest.mark.parametrize("cross", [False, True])
@pytest.mark.parametrize("D,H", [(128, 2), (64, 4)])
def test_reverse_mode_through_the_module(pkg, oracle, nr_oracle, dit_oracle, gpu, cross, D, H):
    """loss = <dout, module(x)>: gradients of x, the context and every weight against torch autograd of the oracle.
    Weight gradients are sums over all tokens in 16-bit GEMMs: relative-L2 <= 2e-2."""
    B, Mq, Mk, K, Kc = 2, 150, 40, 256, (96 if cross else None)
    m = build(pkg, gpu, K, Kc, H, D, torch.bfloat16, 17).train()
    g = torch.Generator().manual_seed(18)
    x = torch.randn(B, Mq, K, generator=g).bfloat16()
    context = torch.randn(B, Mk, Kc, generator=g).bfloat16() if cross else None
    dout = torch.randn(B, Mq, K, generator=g).bfloat16()
    angles = torch.from_numpy(nr_oracle.rope_angles_3d(1, 1, Mq, D))
    xd = x.to(gpu).requires_grad_(True)
    cd = None if context is None else context.to(gpu).requires_grad_(True)
    out = m(xd, cd, rope_emb=angles.reshape(Mq, 1, 1, D).to(gpu))
    out.backward(dout.to(gpu))
    torch.cuda.synchronize()
    want = dit_oracle.attention_module_grads_torch(m.state_dict(), x, dout, context, angles.numpy(), H, D)
    check(oracle, "dx", xd.grad, want["x"])
    if cross:
        check(oracle, "dcontext", cd.grad, want["context"])
    for name, prm in m.named_parameters():
        ma, rl = oracle.error_metrics(prm.grad.float().cpu(), want[name])
        print(f"  d{name}: max_abs={ma:.3e} rel_l2={rl:.3e}", flush=True)
        assert rl <= 2e-2, (name, rl)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_reference_self_attention_procedure(pkg, gpu, dtype):
    """The reference's own live test of the module (context_parallel_test.py:64-91, backends torch / transformer_engine),
    restated for backend "hip": same sizes, same procedure (module output against an explicit softmax(q k^T / sqrt(d)) v
    on the q, k, v that compute_qkv returns, then output_proj), same tolerance atol = rtol = 5e-3.  The module runs in
    16 bits here (the HIP kernels' types); the explicit path is evaluated in fp32 on those 16-bit q, k, v."""
    torch.manual_seed(0)
    batch_size, sequence_length, query_dim, n_heads, head_dim = 2, 16, 64, 4, 32
    attn = pkg.Attention(query_dim=query_dim, n_heads=n_heads, head_dim=head_dim, backend="hip").to(device=gpu, dtype=dtype)
    x_B_S_Q = torch.randn(batch_size, sequence_length, query_dim, device=gpu).to(dtype)
    with torch.no_grad():
        y_B_S_Q = attn(x_B_S_Q)
        assert x_B_S_Q.shape == y_B_S_Q.shape
        q, k, v = (t.float() for t in attn.compute_qkv(x_B_S_Q))
        q, k, v = (t.permute(0, 2, 1, 3) for t in (head_dim ** -0.5 * q, k, v))          # B H S D
        z = (q @ k.transpose(-2, -1)).softmax(dim=-1) @ v
        z_B_S_Q = z.permute(0, 2, 1, 3).reshape(batch_size, sequence_length, n_heads * head_dim) @ attn.output_proj.weight.float().T
    torch.testing.assert_close(y_B_S_Q.float(), z_B_S_Q, atol=5e-3, rtol=5e-3)


def test_fixed_context_is_packed_once_and_reused(pkg, gpu, monkeypatch):
    """Cross-attention against a context tensor that stays the same: its keys / values are projected, normalised and re-tiled
    on the first call only; later calls (forward and forward mode) reuse the image and give the same bits as a module with the
    cache turned off.  A change of the context (in place, or another tensor) or of a weight makes a new image."""
    import copy
    m = build(pkg, gpu, 256, 96, 2, 128, torch.bfloat16, seed=3)
    ref = copy.deepcopy(m)          # the cache is not part of a copy
    ref.cache_context = False
    g = torch.Generator().manual_seed(4)
    x = torch.randn(2, 300, 256, generator=g).to(gpu, torch.bfloat16)
    tx = (torch.randn(2, 300, 256, generator=g) * 0.3).to(gpu, torch.bfloat16)
    context = torch.randn(2, 48, 96, generator=g).to(gpu, torch.bfloat16)
    calls = []
    real_pack = pkg.ops.pack_kv
    monkeypatch.setattr(pkg.ops, "pack_kv", lambda k, v: (calls.append(1), real_pack(k, v))[1])

    def both(mod, ctx):
        with torch.no_grad():
            out = mod(x, ctx)
        out2, tout = mod.forward_jvp(x, tx, ctx)
        return out, out2, tout

    a = both(m, context)
    assert len(calls) == 1                                   # forward packed it, forward mode reused it
    b = both(m, context)
    assert len(calls) == 1
    r = both(ref, context)
    assert len(calls) == 3                                   # cache off: every call packs
    for x1, x2, x3 in zip(a, b, r):
        assert torch.equal(x1, x2) and torch.equal(x1, x3)
    # (forward only and forward + JVP are different kernels, whose workgroups may walk the key tiles in different cyclic
    # orders: the primal outputs agree to rounding, not bit for bit)
    torch.testing.assert_close(a[0].float(), a[1].float(), atol=1e-2, rtol=2e-2)
    context.mul_(0.5)                                        # same tensor, new contents
    c = both(m, context)
    assert len(calls) == 4 and not torch.equal(c[0], a[0])
    assert all(torch.equal(u, w) for u, w in zip(c, both(ref, context)))
    n = len(calls)
    other = context.clone()                                  # another tensor with the same contents
    d = both(m, other)
    assert len(calls) == n + 1 and all(torch.equal(u, w) for u, w in zip(c, d))
    with torch.no_grad():
        m.k_proj.weight.mul_(1.5)
        ref.k_proj.weight.mul_(1.5)
    n = len(calls)
    e = both(m, other)
    assert len(calls) == n + 1 and not torch.equal(e[0], d[0])
    assert all(torch.equal(u, w) for u, w in zip(e, both(ref, other)))
    # with a graph being recorded the module does not use the cache (k, v must stay in the graph)
    n = len(calls)
    xg = x.clone().requires_grad_(True)
    m(xg, other).float().sum().backward()
    assert len(calls) == n and xg.grad is not None


def test_context_made_in_inference_mode(pkg, gpu):
    """The reference makes the text context under ``torch.inference_mode()`` (inference/get_t5_emb.py:50): such tensors have
    no version counter, so the module re-tiles them per call instead of caching, and gives the same bits as with the cache off."""
    import copy
    m = build(pkg, gpu, 256, 96, 2, 128, torch.bfloat16, seed=5)
    ref = copy.deepcopy(m)
    ref.cache_context = False
    g = torch.Generator().manual_seed(6)
    x = torch.randn(1, 200, 256, generator=g).to(gpu, torch.bfloat16)
    tx = (torch.randn(1, 200, 256, generator=g) * 0.3).to(gpu, torch.bfloat16)
    with torch.inference_mode():
        context = torch.randn(1, 40, 96, generator=g).to(gpu, torch.bfloat16) * 1.0
    assert context.is_inference()
    for mode in (torch.no_grad, torch.inference_mode):
        with mode():
            a = m(x, context)
            b = ref(x, context)
        assert torch.equal(a, b)
    a2, ta = m.forward_jvp(x, tx, context)
    b2, tb = ref.forward_jvp(x, tx, context)
    assert torch.equal(a2, b2) and torch.equal(ta, tb)
    assert not m._context_cache                               # nothing was kept for the inference tensor


def test_image_conditioned_cross_attention_cache_matches_uncached(pkg, gpu, monkeypatch):
    """``I2VCrossAttention``: the packed text and image contexts (slots "text" and "image") are reused across forward and
    forward mode, and the results equal those of the same module with the cache turned off; switching the autocast dtype
    over the same context re-tiles instead of tripping on the cached image's dtype."""
    import copy
    torch.manual_seed(7)
    m = pkg.I2VCrossAttention(256, 96, n_heads=2, head_dim=128, img_latent_dim=64)
    m.init_weights()
    m = m.to(device=gpu, dtype=torch.bfloat16).eval()
    ref = copy.deepcopy(m)
    ref.cache_context = False
    g = torch.Generator().manual_seed(8)
    x = torch.randn(2, 260, 256, generator=g).to(gpu, torch.bfloat16)
    tx = (torch.randn(2, 260, 256, generator=g) * 0.3).to(gpu, torch.bfloat16)
    ctx = (torch.randn(2, 48, 96, generator=g).to(gpu, torch.bfloat16), torch.randn(2, 20, 64, generator=g).to(gpu, torch.bfloat16))
    calls = []
    real_pack = pkg.ops.pack_kv
    monkeypatch.setattr(pkg.ops, "pack_kv", lambda k, v: (calls.append(1), real_pack(k, v))[1])
    with torch.no_grad():
        a = m(x, ctx)
    a2, ta = m.forward_jvp(x, tx, ctx)
    assert len(calls) == 2                                    # text + image, packed once for both calls
    with torch.no_grad():
        b = ref(x, ctx)
    b2, tb = ref.forward_jvp(x, tx, ctx)
    assert len(calls) == 6
    assert torch.equal(a, b) and torch.equal(a2, b2) and torch.equal(ta, tb)
    n = len(calls)
    mf = copy.deepcopy(m).float()                             # fp32 weights under two autocast dtypes over one context
    cf = tuple(c.float() for c in ctx)
    for dt in (torch.bfloat16, torch.float16, torch.bfloat16):
        with torch.no_grad(), torch.autocast("cuda", dtype=dt):
            y = mf(x.float(), cf)
        assert y.dtype == dt and torch.isfinite(y.float()).all()
    assert len(calls) == n + 6
