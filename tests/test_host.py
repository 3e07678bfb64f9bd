"""Host-side checks that need no GPU: the C-ABI library loads and exports what the header declares, descriptor
validation returns the documented status codes (validation happens before anything touches the device), and the
Python operators raise the same exception types as the reference for the same misuse."""
import ctypes
import os
import re

import pytest
import torch

import __graft_entry__ as entry

HEADER = os.path.join(entry.REPO_ROOT, "include", "cosmos_attn_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    return re.findall(r"COSMOS_ATTN_API\s+[\w\s\*]+?\b(cosmos_(?:attn|norm|ln|gated|gelu)\w*)\s*\(", text)


def test_header_and_binding_agree(pkg):
    syms = declared_symbols()
    assert len(syms) >= 9
    assert sorted(syms) == sorted(pkg._lib.EXPORTS)


def test_library_exports_every_declared_symbol(pkg):
    lib = ctypes.CDLL(pkg._lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), name
    assert pkg._lib.load_library().cosmos_attn_abi_version() == pkg._lib.ABI_VERSION
    m = re.search(r"#define COSMOS_ATTN_ABI_VERSION (\d+)", open(HEADER).read())
    assert int(m.group(1)) == pkg._lib.ABI_VERSION


def test_desc_struct_layout_matches_header(pkg):
    # 10 x int32/float, 6 pointers, 9 int64, 2 pointers, 3 int64, 2 pointers
    assert ctypes.sizeof(pkg._lib.AttnDesc) == 40 + 6 * 8 + 9 * 8 + 2 * 8 + 3 * 8 + 2 * 8
    assert pkg._lib.AttnDesc.q.offset == 40 and pkg._lib.AttnDesc.key_lens.offset == 208


def good_desc(pkg, **over):
    D = pkg._lib.AttnDesc()
    D.abi_version, D.dtype = pkg._lib.ABI_VERSION, pkg._lib.DTYPE_BF16
    D.B, D.H, D.Lq, D.Lkv, D.d_qk, D.d_v, D.causal, D.sm_scale = 1, 2, 100, 70, 128, 64, 0, 0.1
    fake = 0x7F0000000000  # never dereferenced: validation only looks at values
    D.q, D.k, D.v, D.o = fake, fake + 4096, fake + 8192, fake + 12288
    D.tq = D.tk = D.tv = D.to = None
    for name, sl in (("q_stride", (2 * 100 * 128, 100 * 128, 128)), ("k_stride", (2 * 70 * 128, 70 * 128, 128)),
                     ("v_stride", (2 * 70 * 64, 70 * 64, 64)), ("o_stride", (2 * 100 * 64, 100 * 64, 64))):
        setattr(D, name, (ctypes.c_int64 * 3)(*sl))
    for key, val in over.items():
        setattr(D, key, val)
    return D


def test_status_codes_for_bad_descriptors(pkg):
    L, lib = pkg._lib, pkg._lib.load_library()
    ws = lambda D: lib.cosmos_attn_workspace_bytes(ctypes.byref(D))
    run = lambda D: lib.cosmos_attn_fwd_jvp(ctypes.byref(D), None, 0, None)
    D = good_desc(pkg)
    # forward only: tiles of 32 keys, K part 8 KB + V part (64 -> 2 row blocks) 4 KB
    assert ws(D) == 1 * 2 * 3 * (8 + 4) * 1024
    assert run(D) == L.ST_WORKSPACE          # valid descriptor, no workspace: refused before any launch
    fake = 0x7F0000100000
    assert ws(good_desc(pkg, tq=fake, tk=fake, tv=fake, to=fake)) == 1 * 2 * 3 * 2 * (8 + 4) * 1024
    cases = [
        (dict(abi_version=99), L.ST_BAD_ARG),
        (dict(Lq=0), L.ST_BAD_ARG),
        (dict(q=None), L.ST_BAD_ARG),
        (dict(tk=fake), L.ST_BAD_ARG),                 # tangent on k without q, v
        (dict(tq=fake), L.ST_BAD_ARG),                 # tangents given but no `to`
        (dict(dtype=7), L.ST_UNSUPPORTED),
        (dict(d_qk=512), L.ST_BAD_SHAPE),
        (dict(d_v=48), L.ST_BAD_SHAPE),
        (dict(causal=1), L.ST_BAD_SHAPE),              # causal needs Lq == Lkv
        (dict(q=0x7F0000000008), L.ST_BAD_STRIDE),     # 8-byte aligned base
        (dict(k_stride=(ctypes.c_int64 * 3)(70 * 132, 70 * 132, 132)), L.ST_BAD_STRIDE),
    ]
    for over, want in cases:
        D = good_desc(pkg, **over)
        assert ws(D) == 0, over
        assert run(D) == want, (over, run(D))
        assert lib.cosmos_attn_pack_kv(ctypes.byref(D), None, 0, None) == want
        assert lib.cosmos_attn_run(ctypes.byref(D), None, 0, None) == want
    for st in range(7):
        assert len(L.status_string(st)) > 0
    assert L.status_string(0) == "ok"


def good_bwd_desc(pkg, **over):
    D = pkg._lib.AttnBwdDesc()
    D.abi_version, D.dtype = pkg._lib.ABI_VERSION, pkg._lib.DTYPE_BF16
    D.B, D.H, D.Lq, D.Lkv, D.d, D.causal, D.sm_scale, D.max_ds_mib = 1, 2, 100, 70, 64, 0, 0.1, 0
    fake = 0x7F0000000000  # never dereferenced: validation only looks at values
    for i, name in enumerate(("q", "k", "v", "o", "dout", "lse", "dq", "dk", "dv")):
        setattr(D, name, fake + 4096 * i)
    for name, L in (("q", 100), ("k", 70), ("v", 70), ("o", 100), ("dout", 100), ("dq", 100), ("dk", 70), ("dv", 70)):
        setattr(D, name + "_stride", (ctypes.c_int64 * 3)(2 * L * 64, L * 64, 64))
    for key, val in over.items():
        setattr(D, key, val)
    return D


def test_bwd_desc_layout_and_status_codes(pkg):
    L, lib = pkg._lib, pkg._lib.load_library()
    # 10 x int32/float, 9 pointers, 8 x 3 int64
    assert ctypes.sizeof(L.AttnBwdDesc) == 40 + 9 * 8 + 8 * 3 * 8
    assert L.AttnBwdDesc.q.offset == 40 and L.AttnBwdDesc.dv_stride.offset == 40 + 9 * 8 + 7 * 3 * 8
    ws = lambda D: lib.cosmos_attn_bwd_workspace_bytes(ctypes.byref(D))
    run = lambda D: lib.cosmos_attn_bwd(ctypes.byref(D), None, 0, None)
    D = good_bwd_desc(pkg)
    # statistics (2 floats per query, rounded up to 1 KB) + query stream (4 tiles of 2*4 + 4*2 + 1 fragments)
    # + key stream (3 tiles of 2*4 + 2*2 fragments), per (b, h)
    assert ws(D) == 2048 + 2 * 4 * 17 * 1024 + 2 * 3 * 12 * 1024
    assert run(D) == L.ST_WORKSPACE
    cases = [
        (dict(abi_version=1), L.ST_BAD_ARG),
        (dict(Lkv=0), L.ST_BAD_ARG),
        (dict(lse=None), L.ST_BAD_ARG),
        (dict(dk=None), L.ST_BAD_ARG),
        (dict(dtype=5), L.ST_UNSUPPORTED),
        (dict(d=512), L.ST_BAD_SHAPE),
        (dict(d=48), L.ST_BAD_SHAPE),
        (dict(causal=1), L.ST_BAD_SHAPE),
        (dict(dout=0x7F0000000004), L.ST_BAD_STRIDE),
        (dict(dq_stride=(ctypes.c_int64 * 3)(100 * 66, 100 * 66, 66)), L.ST_BAD_STRIDE),
    ]
    for over, want in cases:
        D = good_bwd_desc(pkg, **over)
        assert ws(D) == 0, over
        assert run(D) == want, (over, run(D))


def test_backward_argument_checks_mirror_reference(pkg):
    q = torch.zeros(1, 2, 8, 64, dtype=torch.bfloat16)
    lse = torch.zeros(1, 2, 8)
    with pytest.raises(AssertionError, match="different headdim"):   # …jvp_triton.py:507-509
        pkg.bwd(q, q, q[..., :32], q, lse, q)
    with pytest.raises(RuntimeError, match="GPU"):                   # no CPU path, no fallback
        pkg.bwd(q, q, q, q, lse, q)
    with pytest.raises(AssertionError, match="Causal cross-attention"):
        pkg.bwd(q, q[:, :, :4], q[:, :, :4], q, lse, q, causal=True)


def test_norm_rope_desc_layout_and_status_codes(pkg):
    L, lib = pkg._lib, pkg._lib.load_library()
    # 8 x int32/float, 6 pointers, 2 x 3 int64
    assert ctypes.sizeof(L.NormRopeDesc) == 32 + 6 * 8 + 2 * 3 * 8
    assert L.NormRopeDesc.x.offset == 32 and L.NormRopeDesc.y_stride.offset == 32 + 6 * 8 + 3 * 8

    def desc(**over):
        D = L.NormRopeDesc()
        D.abi_version, D.dtype, D.B, D.S, D.H, D.D, D.eps = L.ABI_VERSION, L.DTYPE_BF16, 1, 4, 2, 64, 1e-6
        D.x, D.y = 0x7F0000000000, 0x7F0000100000   # never dereferenced: every case below is rejected on the host
        D.x_stride = D.y_stride = (ctypes.c_int64 * 3)(4 * 2 * 64, 2 * 64, 64)
        for k, v in over.items():
            setattr(D, k, v)
        return D

    cases = [
        (dict(abi_version=1), L.ST_BAD_ARG),
        (dict(S=0), L.ST_BAD_ARG),
        (dict(y=None), L.ST_BAD_ARG),
        (dict(tx=0x7F0000200000), L.ST_BAD_ARG),          # a tangent in without a tangent out
        (dict(eps=-1.0), L.ST_BAD_ARG),
        (dict(dtype=5), L.ST_UNSUPPORTED),
        (dict(D=512), L.ST_BAD_SHAPE),
        (dict(D=48), L.ST_BAD_SHAPE),
        (dict(x=0x7F0000000004), L.ST_BAD_STRIDE),
        (dict(angles=0x7F0000300008), L.ST_BAD_STRIDE),
        (dict(y_stride=(ctypes.c_int64 * 3)(4 * 2 * 66, 2 * 66, 66)), L.ST_BAD_STRIDE),
    ]
    for over, want in cases:
        got = lib.cosmos_norm_rope(ctypes.byref(desc(**over)), None)
        assert got == want, (over, got)


def test_norm_rope_bwd_desc_layout_and_status_codes(pkg):
    L, lib = pkg._lib, pkg._lib.load_library()
    # 8 x int32/float, 6 pointers, 3 x 3 int64
    assert ctypes.sizeof(L.NormRopeBwdDesc) == 32 + 6 * 8 + 3 * 3 * 8
    assert L.NormRopeBwdDesc.x.offset == 32 and L.NormRopeBwdDesc.dx_stride.offset == 32 + 6 * 8 + 2 * 3 * 8

    def desc(**over):
        D = L.NormRopeBwdDesc()
        D.abi_version, D.dtype, D.B, D.S, D.H, D.D, D.eps = L.ABI_VERSION, L.DTYPE_BF16, 2, 100, 6, 64, 1e-6
        D.x, D.dy, D.dx, D.dweight = 0x7F0000000000, 0x7F0000100000, 0x7F0000200000, 0x7F0000300000   # never dereferenced
        D.x_stride = D.dy_stride = D.dx_stride = (ctypes.c_int64 * 3)(100 * 6 * 64, 6 * 64, 64)
        for k, v in over.items():
            setattr(D, k, v)
        return D

    ws = lambda D: lib.cosmos_norm_rope_bwd_workspace_bytes(ctypes.byref(D))
    run = lambda D: lib.cosmos_norm_rope_bwd(ctypes.byref(D), None, 0, None)
    # 2 x 100 positions x 2 groups of 4 heads = 400 thread groups, 32 per block (8 threads per row of 64) -> 13 blocks x 64 floats
    assert ws(desc()) == 13 * 64 * 4
    assert ws(desc(dweight=None)) == 0
    assert run(desc()) == L.ST_WORKSPACE
    cases = [
        (dict(abi_version=1), L.ST_BAD_ARG),
        (dict(H=0), L.ST_BAD_ARG),
        (dict(dy=None), L.ST_BAD_ARG),
        (dict(dtype=5), L.ST_UNSUPPORTED),
        (dict(D=512), L.ST_BAD_SHAPE),
        (dict(D=24), L.ST_BAD_SHAPE),
        (dict(dx=0x7F0000200008), L.ST_BAD_STRIDE),
        (dict(dy_stride=(ctypes.c_int64 * 3)(100 * 6 * 66, 6 * 66, 66)), L.ST_BAD_STRIDE),
    ]
    for over, want in cases:
        D = desc(**over)
        assert ws(D) == 0, over
        assert run(D) == want, (over, run(D))


def test_norm_rope_argument_checks(pkg):
    x = torch.zeros(1, 8, 2, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):                   # no CPU path, no fallback
        pkg.norm_rope(x)
    with pytest.raises(AssertionError):
        pkg.norm_rope(x[0])
    with pytest.raises(AssertionError):
        pkg.norm_rope(x, weight=torch.ones(32))
    with pytest.raises(AssertionError, match="one angle per"):
        pkg.norm_rope(x, rope_emb=torch.zeros(4, 1, 1, 64))
    with pytest.raises(AssertionError):                              # head dim outside {16, 32, 64, 128, 256}
        pkg.norm_rope(torch.zeros(1, 8, 2, 48, dtype=torch.bfloat16))


def test_dit_attention_module_mirrors_reference_surface(pkg):
    """Constructor arguments, sub-module / parameter names (a reference state dict must load) and refusals."""
    m = pkg.Attention(64, None, n_heads=2, head_dim=16)
    assert m.is_selfattn and m.backend == "hip"
    # parameter names of cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:349-359 (te RMSNorm holds `weight`)
    assert sorted(m.state_dict()) == ["k_norm.weight", "k_proj.weight", "output_proj.weight", "q_norm.weight",
                                      "q_proj.weight", "v_proj.weight"]
    assert m.q_proj.weight.shape == (32, 64) and m.output_proj.weight.shape == (64, 32) and m.q_norm.weight.shape == (16,)
    c = pkg.Attention(64, 48, n_heads=2, head_dim=16)
    assert not c.is_selfattn and c.k_proj.weight.shape == (32, 48)
    m.init_weights()
    assert float(m.q_proj.weight.abs().max()) <= 3 / 8 + 1e-6 and torch.equal(m.q_norm.weight, torch.ones(16))
    for name in ("compute_qkv", "compute_attention", "forward", "set_context_parallel_group", "init_weights", "forward_jvp"):
        assert callable(getattr(m, name))
    with pytest.raises(AssertionError, match="Invalid backend"):
        pkg.Attention(64, backend="transformer_engine")
    assert isinstance(pkg.Attention(64, backend="minimal_a2a").attn_op, pkg.HipAttnOp)    # the reference's name for this op protocol
    assert pkg.Attention(64, use_wan_fp32_strategy=True).use_wan_fp32_strategy
    with pytest.raises(RuntimeError, match="GPU"):          # no CPU path
        with torch.no_grad():
            m.bfloat16()(torch.zeros(1, 4, 64, dtype=torch.bfloat16))


def test_block_elementwise_desc_layouts_and_status_codes(pkg):
    L, lib = pkg._lib, pkg._lib.load_library()
    assert ctypes.sizeof(L.LnModulateDesc) == 24 + 8 + 8 * 8 and L.LnModulateDesc.x.offset == 32
    assert ctypes.sizeof(L.GatedResidualDesc) == 16 + 8 + 8 * 8 and L.GatedResidualDesc.x.offset == 24
    assert ctypes.sizeof(L.GeluDesc) == 8 + 8 + 4 * 8 and L.GeluDesc.h.offset == 16
    P = 0x7F0000000000   # never dereferenced: every case below is rejected on the host

    def ln(**over):
        D = L.LnModulateDesc()
        D.abi_version, D.dtype, D.D, D.rows_per_group, D.eps, D.rows = L.ABI_VERSION, L.DTYPE_BF16, 256, 4, 1e-6, 16
        D.x, D.shift, D.scale, D.y = P, P + 0x10000, P + 0x20000, P + 0x30000
        for k, v in over.items():
            setattr(D, k, v)
        return D

    for over, want in [(dict(abi_version=1), L.ST_BAD_ARG), (dict(rows=0), L.ST_BAD_ARG), (dict(scale=None), L.ST_BAD_ARG),
                       (dict(tx=P + 0x40000), L.ST_BAD_ARG), (dict(tshift=P + 0x40000), L.ST_BAD_ARG), (dict(dtype=7), L.ST_UNSUPPORTED),
                       (dict(D=8200), L.ST_UNSUPPORTED), (dict(D=252), L.ST_BAD_SHAPE), (dict(rows_per_group=5), L.ST_BAD_SHAPE),
                       (dict(y=P + 0x30002), L.ST_BAD_STRIDE)]:
        assert lib.cosmos_ln_modulate(ctypes.byref(ln(**over)), None) == want, over

    def gr(**over):
        D = L.GatedResidualDesc()
        D.abi_version, D.dtype, D.D, D.rows_per_group, D.rows = L.ABI_VERSION, L.DTYPE_FP16, 64, 2, 8
        D.x, D.res, D.gate, D.out = P, P + 0x10000, P + 0x20000, P
        for k, v in over.items():
            setattr(D, k, v)
        return D

    for over, want in [(dict(abi_version=0), L.ST_BAD_ARG), (dict(gate=None), L.ST_BAD_ARG), (dict(tx=P + 0x40000), L.ST_BAD_ARG),
                       (dict(tgate=P + 0x40000), L.ST_BAD_ARG), (dict(dtype=3), L.ST_UNSUPPORTED), (dict(D=60), L.ST_BAD_SHAPE),
                       (dict(rows=7), L.ST_BAD_SHAPE), (dict(res=P + 8), L.ST_BAD_STRIDE)]:
        assert lib.cosmos_gated_residual(ctypes.byref(gr(**over)), None) == want, over

    def ge(**over):
        D = L.GeluDesc()
        D.abi_version, D.dtype, D.n, D.h, D.a = L.ABI_VERSION, L.DTYPE_BF16, 64, P, P
        for k, v in over.items():
            setattr(D, k, v)
        return D

    for over, want in [(dict(abi_version=0), L.ST_BAD_ARG), (dict(n=0), L.ST_BAD_ARG), (dict(th=P + 0x100), L.ST_BAD_ARG),
                       (dict(dtype=9), L.ST_UNSUPPORTED), (dict(n=12), L.ST_BAD_SHAPE), (dict(a=P + 4), L.ST_BAD_STRIDE)]:
        assert lib.cosmos_gelu(ctypes.byref(ge(**over)), None) == want, over
    with pytest.raises(RuntimeError, match="GPU"):       # no CPU path
        pkg.gelu(torch.zeros(8, dtype=torch.bfloat16))


def test_dit_block_mirrors_reference_surface(pkg):
    m = pkg.Block(64, 48, 2, mlp_ratio=4.0, use_adaln_lora=True, adaln_lora_dim=8)
    names = sorted(m.state_dict())
    # parameter names of cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:1029-1082 (LayerNorms carry none)
    assert names == sorted(
        [f"{a}.{p}.weight" for a in ("self_attn", "cross_attn") for p in ("q_proj", "k_proj", "v_proj", "output_proj", "q_norm", "k_norm")]
        + ["mlp.layer1.weight", "mlp.layer2.weight"]
        + [f"adaln_modulation_{n}.{i}.weight" for n in ("self_attn", "cross_attn", "mlp") for i in (1, 2)])
    assert m.mlp.layer1.weight.shape == (256, 64) and m.adaln_modulation_mlp[2].weight.shape == (192, 8)
    assert m.cross_attn.k_proj.weight.shape == (64, 48) and m.self_attn.is_selfattn and not m.cross_attn.is_selfattn
    m.init_weights()
    assert float(m.adaln_modulation_mlp[2].weight.abs().max()) == 0.0       # the block starts as the identity
    plain = pkg.Block(64, 48, 2)
    assert sorted(k for k in plain.state_dict() if k.startswith("adaln")) == [f"adaln_modulation_{n}.1.weight" for n in ("cross_attn", "mlp", "self_attn")]
    for name in ("forward", "forward_jvp", "init_weights", "reset_parameters", "set_context_parallel_group"):
        assert callable(getattr(m, name))
    i2v = pkg.Block(64, 48, 2, image_context_dim=32)
    assert isinstance(i2v.cross_attn, pkg.I2VCrossAttention) and i2v.cross_attn.k_img.weight.shape == (64, 32)
    assert {"cross_attn.k_img.weight", "cross_attn.v_img.weight", "cross_attn.k_img_norm.weight"} <= set(i2v.state_dict())
    fp32 = pkg.Block(64, 48, 2, use_wan_fp32_strategy=True)
    assert fp32.use_wan_fp32_strategy and fp32.self_attn.use_wan_fp32_strategy and fp32.cross_attn.use_wan_fp32_strategy


def test_dit_network_mirrors_reference_surface(pkg):
    """State-dict names of the reference's network (minimal_v4_dit.py:1338-1432) and its host-side pieces, on the CPU."""
    import numpy as np
    from einops import rearrange

    net = pkg.MiniTrainDIT(max_img_h=16, max_img_w=16, max_frames=8, in_channels=3, out_channels=5, patch_spatial=2, patch_temporal=1,
                           model_channels=64, num_blocks=2, num_heads=2, crossattn_emb_channels=48, use_adaln_lora=True, adaln_lora_dim=8,
                           extra_per_block_abs_pos_emb=True, use_crossattn_projection=True, crossattn_proj_in_channels=40,
                           extra_image_context_dim=24)
    keys = set(net.state_dict())
    for k in ("x_embedder.proj.1.weight", "pos_embedder.seq", "pos_embedder.dim_spatial_range", "pos_embedder.dim_temporal_range",
              "extra_pos_embedder.pos_emb_h", "extra_pos_embedder.pos_emb_w", "extra_pos_embedder.pos_emb_t",
              "t_embedder.1.linear_1.weight", "t_embedder.1.linear_2.weight", "t_embedding_norm.weight",
              "blocks.0.self_attn.q_proj.weight", "blocks.1.cross_attn.k_img_norm.weight", "blocks.1.adaln_modulation_mlp.2.weight",
              "final_layer.linear.weight", "final_layer.adaln_modulation.1.weight", "final_layer.adaln_modulation.2.weight",
              "crossattn_proj.0.weight", "crossattn_proj.0.bias", "img_context_proj.0.weight", "img_context_proj.0.bias"):
        assert k in keys, k
    assert "t_embedder.1.linear_1.bias" not in keys                      # bias only without adaLN-LoRA (:755)
    assert net.x_embedder.proj[1].weight.shape == (64, (3 + 1) * 2 * 2 * 1)    # one more channel for the padding mask
    assert net.t_embedder[1].linear_2.weight.shape == (3 * 64, 64)
    assert net.final_layer.linear.weight.shape == (2 * 2 * 1 * 5, 64)
    assert net.blocks[0].cross_attn.k_img.weight.shape == (64, 64)       # image context is projected to model_channels first
    assert float(net.final_layer.adaln_modulation[2].weight.detach().abs().max()) == 0.0   # init_weights: modulation starts at zero
    plain = pkg.MiniTrainDIT(max_img_h=16, max_img_w=16, max_frames=8, in_channels=3, out_channels=3, patch_spatial=2, patch_temporal=1,
                             model_channels=64, num_blocks=1, num_heads=2, concat_padding_mask=False)
    assert "t_embedder.1.linear_1.bias" in plain.state_dict() and "final_layer.adaln_modulation.2.weight" not in plain.state_dict()
    for kw in (dict(n_dense_blocks=2), dict(natten_parameters={})):
        with pytest.raises(NotImplementedError):
            pkg.MiniTrainDIT(16, 16, 8, 3, 3, 2, 1, model_channels=64, num_blocks=1, num_heads=2, **kw)

    assert not net.is_context_parallel_enabled
    net.enable_context_parallel(None)
    assert net.is_context_parallel_enabled
    net.disable_context_parallel()
    assert not net.is_context_parallel_enabled
    with pytest.raises(NotImplementedError):
        net.fully_shard(None)

    # host-side pieces against einops with the reference's pattern strings / explicit numpy
    x = torch.randn(2, 4, 4, 6, 8)
    pe = pkg.PatchEmbed(2, 2, in_channels=4, out_channels=16)
    want = rearrange(x, "b c (t r) (h m) (w n) -> b t h w (c r m n)", r=2, m=2, n=2) @ pe.proj[1].weight.T
    assert torch.allclose(pe(x), want, atol=1e-6)
    y = torch.randn(2, 3, 4, 4, 2 * 2 * 1 * 5)
    assert torch.equal(net.unpatchify(y), rearrange(y, "B T H W (p1 p2 t C) -> B C (T t) (H p1) (W p2)", p1=2, p2=2, t=1))
    ts = torch.tensor([[0.5, 2.0], [7.0, 0.1]])
    ang = ts.numpy()[..., None].astype(np.float64) * 10000.0 ** (-np.arange(32) / 32)
    assert np.allclose(pkg.Timesteps(64)(ts).numpy(), np.concatenate([np.cos(ang), np.sin(ang)], -1), atol=1e-5)
    emb, lora = net.t_embedder(ts)
    assert emb.shape == (2, 2, 64) and lora.shape == (2, 2, 192) and torch.equal(emb, pkg.Timesteps(64)(ts))
    e = net.extra_pos_embedder(torch.zeros(2, 3, 4, 5, 64))
    raw = (net.extra_pos_embedder.pos_emb_t[:3, None, None] + net.extra_pos_embedder.pos_emb_h[None, :4, None]
           + net.extra_pos_embedder.pos_emb_w[None, None, :5]).detach().double().numpy()
    want = raw / (1e-6 + np.sqrt((raw ** 2).sum(-1, keepdims=True)) / 8.0)
    assert e.shape == (2, 3, 4, 5, 64) and np.allclose(e[1].detach().numpy(), want, atol=1e-5)
    pm = torch.zeros(2, 1, 4, 4)
    pm[:, :, :2] = 1
    xin = net._with_padding_mask(torch.zeros(2, 3, 2, 8, 8), pm)
    assert xin.shape == (2, 4, 2, 8, 8) and float(xin[:, 3, :, :4].min()) == 1.0 and float(xin[:, 3, :, 4:].max()) == 0.0


def test_rope_position_table_mirrors_reference(pkg, nr_oracle):
    """VideoRopePosition3DEmb (cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:534-661): layout, fps and NTK rules."""
    import numpy as np

    T, H, W, D = 3, 4, 5, 128
    pe = pkg.VideoRopePosition3DEmb(head_dim=D, len_h=8, len_w=8, len_t=8)
    assert sorted(pe.state_dict()) == ["dim_spatial_range", "dim_temporal_range", "seq"] and pe.seq_dim == 0
    x = torch.zeros(1, T, H, W, 16)
    e = pe(x, fps=torch.tensor([24.0]))
    assert e.shape == (T * H * W, 1, 1, D) and e.dtype == torch.float32
    # at the base frame rate the table is the plain 3-D one (the oracle's construction, pinned on its own)
    np.testing.assert_allclose(e.reshape(-1, D).numpy(), nr_oracle.rope_angles_3d(T, H, W, D), rtol=1e-6, atol=1e-6)
    # half the frame rate: the temporal angles double (frame index / fps * base_fps), the spatial ones stay
    e12 = pe(x, fps=torch.tensor([12.0])).reshape(T, H, W, D)
    e24 = e.reshape(T, H, W, D)
    dim_h = D // 6 * 2
    dim_t = D - 2 * dim_h
    assert torch.allclose(e12[..., : dim_t // 2], 2 * e24[..., : dim_t // 2]) and torch.equal(e12[..., dim_t // 2: D // 2], e24[..., dim_t // 2: D // 2])
    # image batch: no fps, one frame
    assert pe(torch.zeros(2, 1, H, W, 16)).shape == (H * W, 1, 1, D)
    with pytest.raises(AssertionError, match="T should be 1"):
        pe(x)
    with pytest.raises(AssertionError, match="exceed the maximum"):
        pe(torch.zeros(1, 1, 9, 2, 16))
    # NTK extrapolation: ratio r stretches the base to 10000 * r ** (dim / (dim - 2)) on that axis only
    pe2 = pkg.VideoRopePosition3DEmb(head_dim=D, len_h=8, len_w=8, len_t=8, h_extrapolation_ratio=2.0, enable_fps_modulation=False)
    e2 = pe2(x).reshape(T, H, W, D)
    j = 3                                   # some channel of the h block
    want = 2.0 / (10000.0 * 2.0 ** (dim_h / (dim_h - 2))) ** (2 * j / dim_h)     # position h = 2
    assert abs(float(e2[0, 2, 0, dim_t // 2 + j]) - want) < 1e-6 * want + 1e-9
    assert torch.equal(e2[..., dim_t // 2 + dim_h // 2: D // 2], e24[..., dim_t // 2 + dim_h // 2: D // 2])   # w block untouched
    assert torch.allclose(e2[..., : dim_t // 2], e24[..., : dim_t // 2])            # fps modulation off = base frame rate


def test_status_to_exception_mapping(pkg):
    L = pkg._lib
    L.raise_for_status(L.ST_OK)
    for st, exc in ((L.ST_BAD_SHAPE, AssertionError), (L.ST_BAD_STRIDE, AssertionError), (L.ST_UNSUPPORTED, NotImplementedError),
                    (L.ST_BAD_ARG, ValueError), (L.ST_WORKSPACE, RuntimeError), (L.ST_LAUNCH, RuntimeError)):
        with pytest.raises(exc):
            L.raise_for_status(st)


def test_python_argument_checks_mirror_reference(pkg):
    q = torch.zeros(1, 2, 8, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):          # no CPU path, no fallback
        pkg.fwd_jvp(q, q, q)
    with pytest.raises(AssertionError):                     # shape checks of _attention.forward (…jvp_triton.py:439-440)
        pkg.fwd_jvp(q, q[:, :1], q)
    with pytest.raises(AssertionError):
        pkg.fwd_jvp(q, q, q[:, :, :4])
    with pytest.raises(AssertionError):                     # head dim outside {16,32,64,128,256} (:444-445)
        pkg.fwd_jvp(q[..., :48], q[..., :48], q)
    with pytest.raises(RuntimeError, match="GPU"):          # 256 is built for the forward paths: the call gets as far as the device check
        pkg.fwd_jvp(torch.zeros(1, 1, 8, 256, dtype=torch.bfloat16), torch.zeros(1, 1, 8, 256, dtype=torch.bfloat16),
                    torch.zeros(1, 1, 8, 256, dtype=torch.bfloat16))
    with pytest.raises(AssertionError, match="Causal cross-attention"):   # :446
        pkg.fwd_jvp(q, q[:, :, :4], q[:, :, :4], causal=True)
    with pytest.raises(AssertionError):                     # tangent shape / stride must match the primal (:447-448)
        pkg.attention_jvp(q, q, q, q[:, :, :4], q, q)
    with pytest.raises(AssertionError):
        pkg.attention_jvp(q, q, q, q.transpose(1, 2).contiguous().transpose(1, 2), q, q)
    with pytest.raises(NotImplementedError):                # attention(): dtype not in the supported list (attention.py:107-108)
        pkg.attention_forward(q.transpose(1, 2), q.transpose(1, 2), q.transpose(1, 2), dtype=torch.float64)
    with pytest.raises(NotImplementedError):                # float32 is on the reference's list (SDPA, :145-148) but not built here
        pkg.attention_forward(q.transpose(1, 2), q.transpose(1, 2), q.transpose(1, 2), dtype=torch.float32)


def test_attn_op_refuses_multi_gpu_group(pkg):
    op = pkg.HipAttnOp()
    op.set_context_parallel_group(None, None, None)   # single GPU: accepted, as a2a_cp.py:189-193
    assert op.pg is None


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    r = subprocess.run([sys.executable, os.path.join(entry.REPO_ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_checkpoint_configuration_and_kept_attention_results_bookkeeping(pkg):
    """sac_config parsing (object, dict, enum-valued mode) and the record / replay contexts of attention results: state is
    per thread, restored on exit, and a recomputation that makes fewer attention calls than were recorded is an error."""
    import enum
    import threading
    from types import SimpleNamespace

    class Mode(enum.Enum):
        NONE = "none"
        BLOCK_WISE = "block_wise"

    every = pkg.dit_network._checkpoint_every
    assert every(None) == 0 and every(dict(mode="none")) == 0 and every(SimpleNamespace(mode=Mode.NONE, every_n_blocks=3)) == 0
    assert every(dict(mode="predict2_2b_720_aggressive")) == 1 and every(SimpleNamespace(mode=Mode.BLOCK_WISE, every_n_blocks=2)) == 2
    att = pkg.attention
    store = []
    with att.record_attention_results(store):
        assert att._kept.record is store
        seen = []
        t = threading.Thread(target=lambda: seen.append(att._kept.record))
        t.start(); t.join()
        assert seen == [None]                      # another thread does not record into this one's list
        with att.record_attention_results([]) as inner:
            assert att._kept.record is inner
        assert att._kept.record is store
    assert att._kept.record is None
    with att.replay_attention_results([]):
        assert att._kept.replay == []
    assert att._kept.replay is None
    with pytest.raises(AssertionError, match="fewer attention calls"):
        with att.replay_attention_results([("o", "lse")]):
            pass
    assert att._kept.replay is None
