"""GPU parity: the HIP forward + JVP, called through the C ABI, against the CPU oracle on identical seeded inputs.

Tolerances (16-bit inputs, fp64/fp32 oracle = closed form pinned to torch math SDPA under torch.func.jvp):
max-abs <= 2e-2 and relative-L2 <= 5e-3 for O and dO; LSE max-abs <= 2e-3.
"""
import ctypes
import importlib.util
import math
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ABS, REL_L2, LSE_ABS = 2e-2, 5e-3, 2e-3
GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def check(oracle, name, got, want, max_abs=MAX_ABS, rel_l2=REL_L2):
    ma, rl = oracle.error_metrics(got.float().cpu(), want)
    print(f"  {name}: max_abs={ma:.3e} rel_l2={rl:.3e}", flush=True)
    assert math.isfinite(ma) and ma <= max_abs, f"{name}: max-abs {ma} > {max_abs}"
    assert rl <= rel_l2, f"{name}: rel-L2 {rl} > {rel_l2}"


def run_case(pkg, oracle, gpu, shape_q, shape_kv=None, dv=None, causal=False, sm_scale=None, seed=0,
             dtype=torch.bfloat16, primal_std=1.0, tangent_std=0.1, tangents="full", key_lens=None, rms=False):
    q, k, v, tq, tk, tv = oracle.make_inputs(shape_q, shape_kv, seed=seed, primal_std=primal_std,
                                             tangent_std=tangent_std, rms_norm_qk=rms, dtype=dtype, dv=dv)
    if tangents == "q":
        tk = tv = None
    elif tangents == "none":
        tq = tk = tv = None
    elif tangents == "kv":
        tq = None
    elif tangents == "v":
        tq = tk = None
    print(f"case q={tuple(q.shape)} kv={tuple(k.shape)} dv={v.shape[-1]} causal={causal} dtype={dtype} "
          f"tangents={tangents} key_lens={key_lens} seed={seed}", flush=True)
    dev = lambda x: None if x is None else x.to(gpu)
    kl = None if key_lens is None else torch.tensor(key_lens, dtype=torch.int32, device=gpu)
    o, to, lse = pkg.attention_with_lse(dev(q), dev(k), dev(v), dev(tq), dev(tk), dev(tv), causal=causal,
                                        sm_scale=sm_scale, key_lens=kl)
    torch.cuda.synchronize()
    o_ref, to_ref, lse_ref = oracle.closed_form(q, k, v, tq, tk, tv, sm_scale=sm_scale, causal=causal, key_lens=key_lens)
    check(oracle, "o", o, o_ref)
    if tangents != "none":
        check(oracle, "to", to, to_ref)
    else:
        assert to is None
    ma, _ = oracle.error_metrics(lse.cpu(), lse_ref)
    print(f"  lse: max_abs={ma:.3e}", flush=True)
    assert ma <= LSE_ABS
    return o, to, lse


# ------------------------------------------------------------------ head dims 128 / 128, tangents on k and v, more than 2048 keys
# (past what the query-streaming kernel takes: ragged tails, causal, key padding and key-range splits at that length)
@pytest.mark.parametrize("Lq,Lkv", [(300, 2081), (128, 2112), (517, 4000), (1, 2049), (33, 3000)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_long_key_sequences_full_tangents(pkg, oracle, gpu, Lq, Lkv, dtype):
    run_case(pkg, oracle, gpu, (1, 2, Lq, 128), (1, 2, Lkv, 128), seed=Lq + Lkv, dtype=dtype)


@pytest.mark.parametrize("L", [2049, 2200, 2304])
def test_long_key_sequences_causal(pkg, oracle, gpu, L):
    run_case(pkg, oracle, gpu, (1, 2, L, 128), causal=True, seed=L)


@pytest.mark.parametrize("lens", [[2100, 2600], [1, 2590], [2561, 33]])
def test_long_key_sequences_key_padding(pkg, oracle, gpu, lens):
    run_case(pkg, oracle, gpu, (2, 2, 200, 128), (2, 2, 2600, 128), key_lens=lens, seed=lens[0])


def test_long_key_sequences_key_range_split_and_rms_normed_inputs(pkg, oracle, gpu):
    # 4 (query block, head) pairs on 256 compute units: every pair is cut into 16 key ranges and merged
    run_case(pkg, oracle, gpu, (1, 2, 256, 128), (1, 2, 4096, 128), seed=5, rms=True)
    run_case(pkg, oracle, gpu, (1, 3, 200, 128), (1, 3, 2500, 128), seed=6, tangent_std=1.0)


# ------------------------------------------------------------------ small and ragged shapes
def test_smallest(pkg, oracle, gpu):
    run_case(pkg, oracle, gpu, (1, 1, 64, 128))


@pytest.mark.parametrize("Lq,Lkv", [(1, 1), (50, 37), (31, 33), (129, 1), (5, 300)])
def test_ragged_small(pkg, oracle, gpu, Lq, Lkv):
    run_case(pkg, oracle, gpu, (1, 2, Lq, 128), (1, 2, Lkv, 128), seed=Lq + Lkv)


@pytest.mark.parametrize("L", [128, 192, 999, 1024])
def test_self_attention_d128(pkg, oracle, gpu, L):
    run_case(pkg, oracle, gpu, (1, 2, L, 128), seed=L)


@pytest.mark.parametrize("n_tiles", [1, 2, 3, 4, 5, 7])
@pytest.mark.parametrize("tangents", ["full", "none"])
def test_key_tile_counts(pkg, oracle, gpu, n_tiles, tangents):
    """Whole numbers of 32-key tiles around the LDS ring depths (3 and 4): prologue, wrap-around, drain."""
    run_case(pkg, oracle, gpu, (1, 2, 96, 128), (1, 2, 32 * n_tiles, 128), seed=n_tiles, tangents=tangents)


def test_many_workgroups_rotated_sweeps(pkg, oracle, gpu):
    """64 workgroups per launch: the sweep of a workgroup starts at tile 2 * ((id / 8) mod 32) and wraps around."""
    run_case(pkg, oracle, gpu, (2, 4, 1024, 128), (2, 4, 1500, 128), seed=11)
    run_case(pkg, oracle, gpu, (1, 8, 1024, 64), (1, 8, 700, 64), seed=12, tangents="q")


# ------------------------------------------------------------------ forward only (its own kernel: 384-row workgroups)
@pytest.mark.parametrize("Lq,Lkv", [(1, 1), (50, 37), (383, 65), (385, 64), (129, 1), (5, 300), (800, 96)])
def test_forward_only_ragged(pkg, oracle, gpu, Lq, Lkv):
    run_case(pkg, oracle, gpu, (1, 2, Lq, 128), (1, 2, Lkv, 128), seed=Lq + Lkv, tangents="none")


@pytest.mark.parametrize("dqk,dv", [(16, 16), (32, 128), (64, 64), (128, 32), (128, 16)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_forward_only_head_dims(pkg, oracle, gpu, dqk, dv, dtype):
    run_case(pkg, oracle, gpu, (2, 2, 200, dqk), (2, 2, 333, dqk), dv=dv, seed=dqk + dv, dtype=dtype, tangents="none")


@pytest.mark.parametrize("L", [1, 33, 128, 200, 515, 1000])
def test_forward_only_causal(pkg, oracle, gpu, L):
    run_case(pkg, oracle, gpu, (1, 2, L, 64), causal=True, seed=L, tangents="none")


@pytest.mark.parametrize("lens", [[64, 512], [7, 33], [300, 31], [1, 65]])
def test_forward_only_key_padding(pkg, oracle, gpu, lens):
    run_case(pkg, oracle, gpu, (2, 2, 450, 128), (2, 2, 512, 128), key_lens=lens, seed=sum(lens), tangents="none")


@pytest.mark.parametrize("shape_q,Lkv,ranges", [
    ((1, 2, 1000, 128), 1000, 4),      # 6 workgroup pairs, 16 steps of 64 keys: 4 key ranges each
    ((1, 1, 1157, 32), 4000, 15),      # 4 pairs, 63 steps: 15 ranges of 4 or 5 steps
    ((1, 3, 300, 128), 520, 2),        # 3 pairs, 9 steps: 2 ranges (4 + 5 steps); ragged last tile in the second
    ((2, 8, 6500, 64), 700, 2),        # 272 pairs: 256 whole + 16 cut into ... 11 steps allow 2 ranges
    ((1, 2, 400, 64), 250, 1),         # 4 steps only: too short to cut
])
def test_forward_only_key_range_split(pkg, oracle, gpu, shape_q, Lkv, ranges):
    """When the last round of forward-only workgroups (one per compute unit) is less than half full, its (query block,
    head) pairs are cut along the keys and merged by a second kernel.  The one-call entry point (which may cut) and
    pack + run (which never does) must agree to rounding, and both with the oracle."""
    del ranges   # documented above; the plan itself is internal
    B, H, Lq, d = shape_q
    run_case(pkg, oracle, gpu, shape_q, (B, H, Lkv, d), seed=Lq + Lkv, tangents="none")
    L, lib = pkg._lib, pkg._lib.load_library()
    q, k, v, _, _, _ = (x.to(gpu) for x in oracle.make_inputs(shape_q, (B, H, Lkv, d), seed=Lq + Lkv))
    o_ref, _, lse_ref = pkg.fwd_jvp(q, k, v)
    o, lse = torch.empty_like(q), torch.empty(B, H, Lq, device=gpu)
    D = L.AttnDesc()
    D.abi_version, D.dtype = L.ABI_VERSION, L.DTYPE_BF16
    D.B, D.H, D.Lq, D.Lkv, D.d_qk, D.d_v, D.causal, D.sm_scale = B, H, Lq, Lkv, d, d, 0, d ** -0.5
    D.q, D.k, D.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    s3 = lambda x: (ctypes.c_int64 * 3)(x.stride(0), x.stride(1), x.stride(2))
    D.q_stride, D.k_stride, D.v_stride, D.o_stride = s3(q), s3(k), s3(v), s3(o)
    D.o, D.lse = o.data_ptr(), lse.data_ptr()
    n = lib.cosmos_attn_workspace_bytes(ctypes.byref(D))
    ws = torch.empty(n, device=gpu, dtype=torch.uint8)
    st = torch.cuda.current_stream().cuda_stream
    assert lib.cosmos_attn_pack_kv(ctypes.byref(D), ws.data_ptr(), n, st) == 0
    assert lib.cosmos_attn_run(ctypes.byref(D), ws.data_ptr(), n, st) == 0
    torch.cuda.synchronize()
    assert float((o.float() - o_ref.float()).abs().max()) <= 2.0 ** -7 * max(1.0, float(o_ref.float().abs().max()))
    assert float((lse - lse_ref).abs().max()) <= 1e-4
    # same inputs, same plan: bitwise repeatable
    o_again, _, lse_again = pkg.fwd_jvp(q, k, v)
    assert torch.equal(o_again, o_ref) and torch.equal(lse_again, lse_ref)


@pytest.mark.parametrize("chunk", range(4))
def test_random_shapes_all_modes(pkg, oracle, gpu, chunk):
    """40 seeded random cases (10 per chunk): batch, heads, lengths, head dims, dtype and tangent set drawn at random --
    workgroup counts on either side of the thresholds at which the last round is cut along the keys, key-tile counts
    around the ring depths, ragged ends."""
    rng = np.random.default_rng(1000 + chunk)
    for _ in range(10):
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 13))
        Lq, Lkv = int(rng.integers(1, 1000)), int(rng.integers(1, 1600))
        d = int(rng.choice([16, 32, 64, 128]))
        dv = int(rng.choice([16, 32, 64, 128])) if rng.random() < 0.3 else d
        tangents = str(rng.choice(["full", "q", "none", "kv"]))
        dtype = torch.float16 if rng.random() < 0.3 else torch.bfloat16
        mask = rng.random()
        causal, key_lens = False, None
        if mask < 0.15:
            causal, Lkv = True, Lq
        elif mask < 0.3:
            key_lens = [int(x) for x in rng.integers(1, Lkv + 1, B)]
        run_case(pkg, oracle, gpu, (B, H, Lq, d), (B, H, Lkv, d), dv=dv, causal=causal, key_lens=key_lens,
                 seed=int(rng.integers(0, 10000)), dtype=dtype, tangents=tangents)


def test_against_torch_sdpa_jvp(pkg, oracle, gpu):
    """The quoted oracle itself (torch math SDPA under torch.func.jvp, fp32) on a mid-size case."""
    q, k, v, tq, tk, tv = oracle.make_inputs((2, 3, 300, 128), seed=5)
    o, to = pkg.attention_jvp(*(x.to(gpu) for x in (q, k, v, tq, tk, tv)))
    o_ref, to_ref = oracle.sdpa_jvp_torch(q, k, v, tq, tk, tv)
    check(oracle, "o", o, o_ref)
    check(oracle, "to", to, to_ref)


# ------------------------------------------------------------------ head dims, dtypes, tangent sets
@pytest.mark.parametrize("dqk,dv", [(16, 16), (16, 32), (32, 128), (64, 64), (64, 128), (128, 32), (128, 64), (32, 16), (128, 16)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_head_dims(pkg, oracle, gpu, dqk, dv, dtype):
    run_case(pkg, oracle, gpu, (1, 2, 150, dqk), (1, 2, 170, dqk), dv=dv, dtype=dtype, seed=dqk + dv, primal_std=0.5, tangent_std=0.5)


@pytest.mark.parametrize("dqk,dv", [(256, 256), (256, 64), (128, 256), (16, 256), (256, 16)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tangents", ["full", "q", "none"])
def test_head_dim_256(pkg, oracle, gpu, dqk, dv, dtype, tangents):
    """Head dim 256 (flash_attention_jvp_triton.py:444-445 accepts it) runs a kernel of its own: ragged lengths, more than
    one key tile, every tangent set."""
    run_case(pkg, oracle, gpu, (1, 2, 150, dqk), (1, 2, 77, dqk), dv=dv, dtype=dtype, tangents=tangents, seed=dqk + dv)
    run_case(pkg, oracle, gpu, (2, 1, 33, dqk), (2, 1, 300, dqk), dv=dv, dtype=dtype, tangents=tangents, seed=dqk + dv + 1)


def test_head_dim_256_masks_and_reference_shapes(pkg, oracle, gpu):
    run_case(pkg, oracle, gpu, (1, 2, 200, 256), causal=True, seed=1)
    run_case(pkg, oracle, gpu, (1, 2, 200, 256), causal=True, tangents="none", seed=2)
    run_case(pkg, oracle, gpu, (2, 2, 100, 256), (2, 2, 90, 256), key_lens=[64, 7], tangents="q", seed=3)
    run_case(pkg, oracle, gpu, (1, 2, 1024, 256), seed=4, primal_std=0.5, tangent_std=0.5, sm_scale=0.5)   # the reference's test scale
    # strided [B, L, H, d] views and [B, L, H, d] output memory
    q, k, v, tq, tk, tv = oracle.make_inputs((1, 2, 130, 256), seed=5)
    blhd = lambda x: x.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3).to(gpu)
    o, to, lse = pkg.fwd_jvp(blhd(q), blhd(k), blhd(v), blhd(tq), blhd(tk), blhd(tv), out_layout="blhd")
    o_ref, to_ref, _ = oracle.closed_form(q, k, v, tq, tk, tv)
    check(oracle, "o", o, o_ref)
    check(oracle, "to", to, to_ref)


@pytest.mark.parametrize("tangents", ["none", "q", "kv", "v"])
@pytest.mark.parametrize("dqk,dv", [(128, 128), (64, 32)])
def test_tangent_sets(pkg, oracle, gpu, tangents, dqk, dv):
    run_case(pkg, oracle, gpu, (2, 2, 140, dqk), (2, 2, 100, dqk), dv=dv, tangents=tangents, seed=3)


# ------------------------------------------------------------------ masks
@pytest.mark.parametrize("L", [1, 33, 128, 200, 515])
def test_causal(pkg, oracle, gpu, L):
    run_case(pkg, oracle, gpu, (1, 2, L, 64), causal=True, sm_scale=0.5, primal_std=0.5, tangent_std=0.5, seed=L)


def test_causal_d128_q_only(pkg, oracle, gpu):
    run_case(pkg, oracle, gpu, (2, 2, 300, 128), causal=True, tangents="q", seed=8)


@pytest.mark.parametrize("lens", [[64, 512], [7, 33], [300, 31]])
def test_key_padding(pkg, oracle, gpu, lens):
    Lkv = max(lens) if max(lens) > 100 else 70
    run_case(pkg, oracle, gpu, (2, 2, 200, 128), (2, 2, Lkv, 128), key_lens=lens, tangents="q", seed=sum(lens))
    run_case(pkg, oracle, gpu, (2, 2, 100, 128), (2, 2, Lkv, 128), key_lens=lens, tangents="full", seed=sum(lens) + 1)


def test_single_valid_key(pkg, oracle, gpu):
    """key_lens = 1: O = V[0] and the q-tangent cancels exactly in exact arithmetic (H V - r O with one key).  The kernel
    (like the reference, flash_attention_jvp_triton.py:134-146) rounds H to 16 bits but sums r in fp32, so what is left is
    that rounding: checked in absolute terms (a relative measure against an all-zero answer means nothing)."""
    q, k, v, tq, _, _ = oracle.make_inputs((1, 2, 100, 128), (1, 2, 40, 128), seed=2)
    kl = torch.tensor([1], dtype=torch.int32, device=gpu)
    o, to, lse = pkg.attention_with_lse(q.to(gpu), k.to(gpu), v.to(gpu), tq.to(gpu), key_lens=kl)
    assert torch.equal(o.cpu(), v[:, :, :1].expand_as(o))
    assert to.float().abs().max().item() <= MAX_ABS
    _, _, lse_ref = oracle.closed_form(q, k, v, key_lens=[1])
    assert oracle.error_metrics(lse.cpu(), lse_ref)[0] <= LSE_ABS


# ------------------------------------------------------------------ short key sequences: the query-streaming kernels
# The library sends a call to the streaming kernels only when it has a thousand (query block, head) pairs or more; the
# library's hook cosmos_attn_set_stream_override (query blocks per workgroup; the `stream_override` fixture) forces them on small ones.
@pytest.mark.parametrize("chunk", [2, 3, 16])
@pytest.mark.parametrize("tangents", ["q", "none", "full"])
def test_streaming_kernels_key_tile_counts(pkg, oracle, gpu, stream_override, chunk, tangents):
    stream_override(chunk=chunk)
    for i, Lkv in enumerate([1, 20, 32, 33, 64, 96, 100, 160, 257, 512]):
        if Lkv == 1 and tangents == "q":
            continue   # one key: the q-tangent cancels to rounding noise (test_single_valid_key), a relative measure means nothing
        run_case(pkg, oracle, gpu, (1, 2, 700, 128), (1, 2, Lkv, 128), tangents=tangents, seed=10 * chunk + i)


@pytest.mark.parametrize("tangents", ["q", "none", "full"])
@pytest.mark.parametrize("lens", [[64, 512], [7, 33], [300, 31], [2, 65], [96, 97]])
def test_streaming_kernels_key_padding(pkg, oracle, gpu, stream_override, lens, tangents):
    stream_override(chunk=4)
    Lkv = max(lens) if max(lens) > 100 else 100
    run_case(pkg, oracle, gpu, (2, 3, 1100, 128), (2, 3, Lkv, 128), key_lens=lens, tangents=tangents, seed=sum(lens))


@pytest.mark.parametrize("groups", [8, 40, 256])
@pytest.mark.parametrize("tangents", ["q", "none", "full"])
def test_streaming_kernels_pieces_of_equal_weight(pkg, oracle, gpu, stream_override, groups, tangents):
    """The hook's second argument sets the number of workgroups directly.  The kernel cuts the line of (query block, head)
    pairs into that many pieces of equal weight, a pair weighing by its batch row's key length: with rows of 16, 2 and 7
    key tiles the pieces hold different numbers of blocks, run over head and row boundaries, and with 256 workgroups for
    174 pairs some are empty."""
    stream_override(groups=groups)
    run_case(pkg, oracle, gpu, (3, 2, 900, 128), (3, 2, 512, 128), key_lens=[512, 40, 200], tangents=tangents, seed=groups)


@pytest.mark.parametrize("chunk", [0, 1, 2])
def test_streaming_kernels_random_shapes(pkg, oracle, gpu, stream_override, chunk):
    """36 seeded random cases (12 per chunk) through the streaming kernels: batch, heads, query and key lengths, per-row key
    lengths, head dim, dtype, tangent set and the number of workgroups drawn at random."""
    import random
    rng = random.Random(77 + chunk)
    for it in range(12):
        d = rng.choice([16, 32, 64, 128, 128, 128])
        dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16])
        tangents = rng.choice(["q", "q", "none", "full"])
        B, H = rng.choice([1, 2, 3]), rng.choice([1, 2, 3])
        Lq = rng.choice([1, 37, 128, 129, 300, 640, 777, 1100, 1500])
        Lkv = rng.choice([17, 32, 33, 64, 65, 96, 100, 128, 160, 200, 257, 384, 512, 700])
        lens = [rng.randint(2, Lkv) for _ in range(B)] if rng.random() < 0.5 else None
        stream_override(groups=rng.choice([8, 16, 24, 40, 64, 256]))
        run_case(pkg, oracle, gpu, (B, H, Lq, d), (B, H, Lkv, d), tangents=tangents, dtype=dtype, key_lens=lens,
                 seed=9000 + 100 * chunk + it)


@pytest.mark.parametrize("d", [16, 32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tangents", ["q", "none", "full"])
def test_streaming_kernels_head_dims(pkg, oracle, gpu, stream_override, d, dtype, tangents):
    stream_override(chunk=3)
    run_case(pkg, oracle, gpu, (1, 2, 650, d), (1, 2, 150, d), tangents=tangents, dtype=dtype, seed=d)
    run_case(pkg, oracle, gpu, (1, 2, 129, d), (1, 2, 70, d), tangents=tangents, dtype=dtype, seed=d + 1)


@pytest.mark.parametrize("tangents", ["q", "none"])
def test_streaming_kernels_match_the_block_kernels_bitwise_free(pkg, oracle, gpu, stream_override, tangents):
    """Streamed and not streamed: same arithmetic per tile, but the streaming kernels may walk the tiles in another
    cyclic order and pad a one-tile row with a masked tile, so the results agree to rounding, not bit for bit; both must
    meet the oracle.  Strided (B, L, H, d) views, one query block per workgroup at the end of the stream (1000 rows, 3 per
    workgroup)."""
    q, k, v, tq, _, _ = oracle.make_inputs((2, 2, 1000, 128), (2, 2, 300, 128), seed=5)
    blhd = lambda x: x.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3).to(gpu)   # (B, H, L, d) view of (B, L, H, d) memory
    args = (blhd(q), blhd(k), blhd(v), blhd(tq) if tangents == "q" else None)
    kl = torch.tensor([300, 77], dtype=torch.int32, device=gpu)
    stream_override(chunk=1)
    ref = pkg.attention_with_lse(*args, key_lens=kl)
    stream_override(chunk=3)
    got = pkg.attention_with_lse(*args, key_lens=kl)
    torch.cuda.synchronize()
    o_ref, to_ref, lse_ref = oracle.closed_form(q, k, v, tq if tangents == "q" else None, None, None, key_lens=[300, 77])
    for res in (ref, got):
        check(oracle, "o", res[0], o_ref)
        if tangents == "q":
            check(oracle, "to", res[1], to_ref)
        assert oracle.error_metrics(res[2].cpu(), lse_ref)[0] <= LSE_ABS
    assert (got[0].float() - ref[0].float()).abs().max().item() <= 1e-2


def test_streaming_kernel_reproducible(pkg, oracle, gpu, stream_override):
    stream_override(chunk=5)
    q, k, v, tq, _, _ = oracle.make_inputs((1, 4, 2000, 128), (1, 4, 200, 128), seed=8)
    a = pkg.attention_with_lse(q.to(gpu), k.to(gpu), v.to(gpu), tq.to(gpu))
    b = pkg.attention_with_lse(q.to(gpu), k.to(gpu), v.to(gpu), tq.to(gpu))
    assert all(torch.equal(x, y) for x, y in zip(a, b))


# ------------------------------------------------------------------ the reference's own test shapes
@pytest.mark.parametrize("shape", [(1, 2, 1024, 64), (1, 2, 999, 64)])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reference_jvp_shapes(pkg, oracle, gpu, shape, causal, dtype):
    """flash_attention_jvp_triton.py:610-642: shapes (1,2,1024,64), (1,2,999,64), causal in {T,F}, fp16/bf16,
    N(0,0.5) primals and tangents, sm_scale 0.5, tolerance atol = rtol = 1e-2 on the tangent."""
    o, to, _ = run_case(pkg, oracle, gpu, shape, causal=causal, sm_scale=0.5, primal_std=0.5, tangent_std=0.5, dtype=dtype, seed=20)
    q, k, v, tq, tk, tv = oracle.make_inputs(shape, seed=20, primal_std=0.5, tangent_std=0.5, dtype=dtype)
    o_ref, to_ref, _ = oracle.closed_form(q, k, v, tq, tk, tv, sm_scale=0.5, causal=causal)
    torch.testing.assert_close(o.float().cpu(), torch.from_numpy(o_ref).float(), atol=1e-2, rtol=0)
    torch.testing.assert_close(to.float().cpu(), torch.from_numpy(to_ref).float(), atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("shape", [(1, 2, 256, 1024, 64, 128), (1, 2, 1000, 15, 128, 32), (1, 2, 512, 512, 16, 32), (1, 2, 515, 999, 16, 32),
                                   (1, 2, 256, 1024, 128, 128), (1, 2, 1024, 256, 128, 128), (1, 2, 1024, 512, 64, 64), (1, 2, 1000, 515, 64, 64)])
def test_reference_cross_attention_shapes(pkg, oracle, gpu, shape):
    """flash_attention_jvp_triton.py:803-809 (d_qk != d_v) and :758-759 (cross lengths); out atol 1e-2, tangent atol 2e-2."""
    Z, H, Lq, Lkv, dqk, dv = shape
    run_case(pkg, oracle, gpu, (Z, H, Lq, dqk), (Z, H, Lkv, dqk), dv=dv, sm_scale=0.5, primal_std=0.5, tangent_std=0.5, seed=20)


# ------------------------------------------------------------------ the drop-in surfaces
def test_strided_views_and_blhd_output(pkg, oracle, gpu):
    """[B, S, H, D] tensors handed over as transposed views (no copy), output written in [B, S, H, D] memory."""
    B, S, H, D = 2, 260, 3, 128
    q, k, v, tq, tk, tv = (x.to(gpu) for x in oracle.make_inputs((B, S, H, D), seed=6))
    tr = lambda x: x.transpose(1, 2)
    o, to, lse = pkg.fwd_jvp(tr(q), tr(k), tr(v), tr(tq), tr(tk), tr(tv), out_layout="blhd")
    assert o.shape == (B, H, S, D) and o.transpose(1, 2).is_contiguous() and to.transpose(1, 2).is_contiguous()
    o_ref, to_ref, lse_ref = oracle.closed_form(*(tr(x).cpu() for x in (q, k, v, tq, tk, tv)))
    check(oracle, "o", o, o_ref)
    check(oracle, "to", to, to_ref)
    # a view whose rows are not 16-byte aligned is copied by the host and still gives the same answer
    qo = torch.zeros(B, H, S, D + 4, device=gpu, dtype=q.dtype)[..., 4:]
    qo.copy_(tr(q))
    o2, _, _ = pkg.fwd_jvp(qo, tr(k), tr(v))
    o3, _, _ = pkg.fwd_jvp(tr(q).contiguous(), tr(k), tr(v))
    assert torch.equal(o2, o3)


def test_attention_forward_matches_sdpa(pkg, oracle, gpu):
    """networks/attention.py:90-181 semantics: [B,S,H,D] in, contiguous [B,S,H,D] out, q_scale, softmax_scale, causal."""
    B, S, H, D = 2, 333, 4, 128
    q, k, v, _, _, _ = oracle.make_inputs((B, S, H, D), seed=9, dtype=torch.float32)
    out = pkg.attention_forward(q.to(gpu), k.to(gpu), v.to(gpu))          # cast to bf16 inside, like the reference
    assert out.shape == (B, S, H, D) and out.is_contiguous() and out.dtype == torch.bfloat16
    tr = lambda x: x.to(torch.bfloat16).transpose(1, 2)
    ref = oracle.sdpa_forward_torch(tr(q), tr(k), tr(v)).transpose(1, 2)
    check(oracle, "attention()", out, ref)
    out = pkg.attention_forward(q.to(gpu), k.to(gpu), v.to(gpu), q_scale=0.5, softmax_scale=0.2, causal=True, dtype=torch.float16,
                                deterministic=True, q_lens=None, k_lens=None)
    tr16 = lambda x: x.to(torch.float16).transpose(1, 2)
    ref = oracle.sdpa_forward_torch((q.to(torch.float16) * 0.5).transpose(1, 2), tr16(k), tr16(v), sm_scale=0.2, causal=True).transpose(1, 2)
    check(oracle, "attention(causal, fp16)", out, ref)


def test_attention_forward_refuses_dropout(pkg, oracle, gpu):
    """attention(dropout_p != 0): the reference's SDPA branch (attention.py:170-178), the one a ROCm build takes, applies it; the
    HIP kernels have no dropout and say so instead of returning unregularised attention.  dropout_p = 0 is served."""
    q, k, v, _, _, _ = oracle.make_inputs((1, 2, 200, 128), seed=9)
    bshd = lambda x: x.to(gpu).transpose(1, 2).contiguous()
    pkg.attention_forward(bshd(q), bshd(k), bshd(v), dropout_p=0.0)
    with pytest.raises(NotImplementedError, match="dropout_p"):
        pkg.attention_forward(bshd(q), bshd(k), bshd(v), dropout_p=0.1)


def test_attn_op_protocol(pkg, oracle, gpu):
    """a2a_cp.py:208-219 / minimal_v4_dit.py:252-283: op(q,k,v [B,S,H,D]) -> [B,S,H*D]; cross-attention lengths differ."""
    B, S, H, D, Lc = 2, 200, 4, 128, 77
    q, _, _, tq, _, _ = oracle.make_inputs((B, S, H, D), seed=1)
    k, v, _, _, _, _ = oracle.make_inputs((B, Lc, H, D), seed=2)
    op = pkg.HipAttnOp()
    op.set_context_parallel_group(None, None, None)
    out = op(q.to(gpu), k.to(gpu), v.to(gpu), video_size=(1, 10, 20))
    assert out.shape == (B, S, H * D)
    tr = lambda x: x.transpose(1, 2)
    ref = oracle.sdpa_forward_torch(tr(q), tr(k), tr(v)).transpose(1, 2).reshape(B, S, H * D)
    check(oracle, "HipAttnOp", out, ref)
    assert torch.equal(out, pkg.hip_attention_op(q.to(gpu), k.to(gpu), v.to(gpu)))
    o2, to2 = op.forward_jvp(q.to(gpu), k.to(gpu), v.to(gpu), tq.to(gpu))
    o_ref, to_ref, _ = oracle.closed_form(tr(q), tr(k), tr(v), tr(tq))
    check(oracle, "HipAttnOp.forward_jvp o", o2, np.ascontiguousarray(o_ref.transpose(0, 2, 1, 3)).reshape(B, S, H * D))
    check(oracle, "HipAttnOp.forward_jvp", to2, np.ascontiguousarray(to_ref.transpose(0, 2, 1, 3)).reshape(B, S, H * D))


def test_autograd_function_contract(pkg, oracle, gpu):
    """_attention.apply: positional (q,k,v,tq,tk,tv,causal,sm_scale) -> (o, to); `to` carries no gradient; backward
    runs through o only (tests/test_gpu_backward.py checks the gradients; unequal head dims are refused like the
    reference, …jvp_triton.py:507-509)."""
    q, k, v, tq, tk, tv = (x.to(gpu) for x in oracle.make_inputs((1, 2, 100, 64), seed=3))
    o, to = pkg.attention_jvp(q, k, v, tq, tk, tv, False, 0.25)
    o_ref, to_ref, _ = oracle.closed_form(q.cpu(), k.cpu(), v.cpu(), tq.cpu(), tk.cpu(), tv.cpu(), sm_scale=0.25)
    check(oracle, "o", o, o_ref)
    check(oracle, "to", to, to_ref)
    qg = q.clone().requires_grad_()
    o, to = pkg.attention_jvp(qg, k, v, tq, tk, tv)
    assert o.requires_grad and not to.requires_grad
    o.sum().backward()
    assert qg.grad is not None and qg.grad.shape == q.shape and torch.isfinite(qg.grad.float()).all()
    q2, k2, v2, tq2, tk2, tv2 = (x.to(gpu) for x in oracle.make_inputs((1, 2, 40, 64), (1, 2, 40, 64), seed=3, dv=32))
    o, _ = pkg.attention_jvp(q2.requires_grad_(), k2, v2, tq2, tk2, tv2)
    with pytest.raises(AssertionError, match="different headdim"):
        o.sum().backward()


def test_c_abi_two_stage_equals_one_call(pkg, oracle, gpu):
    """cosmos_attn_pack_kv + cosmos_attn_run called directly through ctypes == cosmos_attn_fwd_jvp; workspace reuse across
    two runs with different q (the cross-attention / fixed-context use)."""
    L, lib = pkg._lib, pkg._lib.load_library()
    q, k, v, tq, _, _ = (x.to(gpu) for x in oracle.make_inputs((1, 2, 300, 128), (1, 2, 77, 128), seed=4))
    o_ref, to_ref, lse_ref = pkg.fwd_jvp(q, k, v, tq)
    o, to = torch.empty_like(q), torch.empty_like(q)
    lse = torch.empty(1, 2, 300, device=gpu)
    D = L.AttnDesc()
    D.abi_version, D.dtype = L.ABI_VERSION, L.DTYPE_BF16
    D.B, D.H, D.Lq, D.Lkv, D.d_qk, D.d_v, D.causal, D.sm_scale = 1, 2, 300, 77, 128, 128, 0, 128 ** -0.5
    D.q, D.k, D.v, D.tq, D.tk, D.tv = q.data_ptr(), k.data_ptr(), v.data_ptr(), tq.data_ptr(), None, None
    s3 = lambda x: (ctypes.c_int64 * 3)(x.stride(0), x.stride(1), x.stride(2))
    D.q_stride, D.k_stride, D.v_stride, D.o_stride = s3(q), s3(k), s3(v), s3(o)
    D.o, D.to, D.lse, D.key_lens = o.data_ptr(), to.data_ptr(), lse.data_ptr(), None
    n = lib.cosmos_attn_workspace_bytes(ctypes.byref(D))
    ws = torch.empty(n, device=gpu, dtype=torch.uint8)
    st = torch.cuda.current_stream().cuda_stream
    assert lib.cosmos_attn_pack_kv(ctypes.byref(D), ws.data_ptr(), n, st) == 0
    assert lib.cosmos_attn_run(ctypes.byref(D), ws.data_ptr(), n, st) == 0
    torch.cuda.synchronize()
    assert torch.equal(o, o_ref) and torch.equal(to, to_ref) and torch.equal(lse, lse_ref)
    q2 = (q * 0.5).contiguous()
    D.q = q2.data_ptr()
    assert lib.cosmos_attn_run(ctypes.byref(D), ws.data_ptr(), n, st) == 0
    torch.cuda.synchronize()
    o2_ref, _, _ = pkg.fwd_jvp(q2, k, v, tq)
    assert torch.equal(o, o2_ref)
    npk = lib.cosmos_attn_packed_bytes(ctypes.byref(D))      # the two-stage calls need the image only
    assert 0 < npk <= n
    assert lib.cosmos_attn_run(ctypes.byref(D), ws.data_ptr(), npk, st) == 0
    assert lib.cosmos_attn_run(ctypes.byref(D), ws.data_ptr(), npk - 1, st) == L.ST_WORKSPACE


def test_hip_graph_capture_and_replay(pkg, oracle, gpu):
    """The entry points launch kernels only (no synchronisation, no memset, no allocation of their own), so a call can be
    captured into a HIP graph; replays with new input contents, with eager work in between, match eager calls bit for bit."""
    make = lambda seed: [x.to(gpu) for x in oracle.make_inputs((1, 2, 300, 128), (1, 2, 200, 128), seed=seed)]
    static = make(0)
    pkg.fwd_jvp(*static)                      # eager warm-up (first call configures the kernels)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        pkg.fwd_jvp(*static)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o_g, to_g, lse_g = pkg.fwd_jvp(*static)
    for seed in (1, 2, 3):
        fresh = make(seed)
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        o_e, to_e, lse_e = pkg.fwd_jvp(*fresh)   # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(o_g, o_e) and torch.equal(to_g, to_e) and torch.equal(lse_g, lse_e), seed


def test_hip_graph_capture_with_key_range_split(pkg, oracle, gpu):
    """The cut of a thin last round (several launches: attention kernel + merge kernel, scratch in the caller's workspace)
    under graph capture: replays match eager calls bit for bit, forward only and forward + JVP."""
    make = lambda seed: [x.to(gpu) for x in oracle.make_inputs((1, 2, 1000, 128), (1, 2, 1000, 128), seed=seed)]
    static = make(0)
    pkg.fwd_jvp(*static); pkg.fwd_jvp(*static[:3])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        pkg.fwd_jvp(*static); pkg.fwd_jvp(*static[:3])
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o_g, to_g, lse_g = pkg.fwd_jvp(*static)
        of_g, _, lsef_g = pkg.fwd_jvp(*static[:3])
    for seed in (1, 2):
        fresh = make(seed)
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        o_e, to_e, lse_e = pkg.fwd_jvp(*fresh)
        of_e, _, lsef_e = pkg.fwd_jvp(*fresh[:3])
        torch.cuda.synchronize()
        assert torch.equal(o_g, o_e) and torch.equal(to_g, to_e) and torch.equal(lse_g, lse_e), seed
        assert torch.equal(of_g, of_e) and torch.equal(lsef_g, lsef_e), seed


def test_golden_fixtures(pkg, oracle, gpu):
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(GOLDEN_DIR, "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    gold = np.load(os.path.join(GOLDEN_DIR, "attn_jvp_golden.npz"))
    for name in mg.CASES:
        (q, k, v, tq, tk, tv), kw = mg.case_inputs(oracle, name)
        if q.dtype == torch.float32:
            # the kernels take 16-bit inputs: the fp32 plumbing case runs on its inputs rounded to bf16 and is held to
            # the same tolerance against the fp32 expectation (the rounding of the inputs is part of the error)
            q, k, v, tq, tk, tv = (x.to(torch.bfloat16) for x in (q, k, v, tq, tk, tv))
        print("golden", name, flush=True)
        kl = None if kw["key_lens"] is None else torch.tensor(kw["key_lens"], dtype=torch.int32, device=gpu)
        o, to, lse = pkg.attention_with_lse(*(x.to(gpu) for x in (q, k, v, tq, tk, tv)), causal=kw["causal"], sm_scale=kw["sm_scale"], key_lens=kl)
        check(oracle, "o", o, gold[name + "/o"])
        check(oracle, "to", to, gold[name + "/to"])
        assert oracle.error_metrics(lse.cpu(), gold[name + "/lse"])[0] <= LSE_ABS


# ------------------------------------------------------------------ the benchmark shapes: sampled row blocks + size-independent properties
def sampled_rows_check(pkg, oracle, gpu, H, Lq, Lkv, tangents, rms, key_lens=None, B=1, seed=0, n_blocks=8):
    """Full-length sequences: the fp32 score matrix cannot exist, so 128-row blocks (first, last / ragged, random) of a
    couple of heads are checked against the row-block oracle -- exact, because query rows are independent."""
    q, k, v, tq, tk, tv = oracle.make_inputs((B, H, Lq, 128), (B, H, Lkv, 128), seed=seed, rms_norm_qk=rms)
    if tangents == "q":
        tk = tv = None
    if tangents == "none":
        tq = tk = tv = None
    dev = lambda x: None if x is None else x.to(gpu)
    kl = None if key_lens is None else torch.tensor(key_lens, dtype=torch.int32, device=gpu)
    o, to, lse = pkg.fwd_jvp(dev(q), dev(k), dev(v), dev(tq), dev(tk), dev(tv), key_lens=kl)
    torch.cuda.synchronize()
    rng = np.random.default_rng(seed)
    starts = [0, max(Lq - 128, 0)] + [int(x) for x in rng.integers(0, max(Lq - 128, 1), n_blocks - 2)]
    for i, r0 in enumerate(starts):
        b, h = i % B, int(rng.integers(0, H))
        rows = slice(r0, min(r0 + 128, Lq))
        sel = lambda x: None if x is None else x[b, h]
        o_ref, to_ref, lse_ref = oracle.rows_oracle(q[b, h, rows], sel(k), sel(v), None if tq is None else tq[b, h, rows], sel(tk), sel(tv),
                                                    kv_len=None if key_lens is None else key_lens[b])
        print(f" rows {r0}..{rows.stop} of (b={b}, h={h})", flush=True)
        check(oracle, "o", o[b, h, rows], o_ref)
        if to is not None:
            check(oracle, "to", to[b, h, rows], to_ref)
        assert oracle.error_metrics(lse[b, h, rows].cpu(), lse_ref)[0] <= LSE_ABS
    return (q, k, v, tq, tk, tv), (o, to, lse)


def test_more_than_2_31_elements(pkg, oracle, gpu):
    """Offsets beyond 32 bits: q, k, v and tangents of 2.2e9 elements each (B=4, H=128, L=32896, d=128), generated on the
    GPU; row blocks of the first and of the last (batch, head) against the row-block oracle, forward + JVP and forward only."""
    B, H, L, d = 4, 128, 32896, 128
    assert B * H * L * d > 2 ** 31
    g = torch.Generator(device=gpu).manual_seed(0)

    def rn(std):
        x = torch.empty(B, H, L, d, device=gpu, dtype=torch.bfloat16)
        for b in range(B):
            x[b] = (torch.randn(H, L, d, generator=g, device=gpu) * std).bfloat16()
        return x

    q, k, v, tq, tk, tv = rn(1.0), rn(1.0), rn(1.0), rn(0.1), rn(0.1), rn(0.1)
    o, to, lse = pkg.fwd_jvp(q, k, v, tq, tk, tv)
    o_f, _, lse_f = pkg.fwd_jvp(q, k, v)
    torch.cuda.synchronize()
    c = lambda x: x.cpu()
    for b, h, r0 in ((0, 0, 0), (B - 1, H - 1, 0), (B - 1, H - 1, L - 128), (2, 77, 12345)):
        rows = slice(r0, r0 + 128)
        o_ref, to_ref, lse_ref = oracle.rows_oracle(c(q[b, h, rows]), c(k[b, h]), c(v[b, h]), c(tq[b, h, rows]), c(tk[b, h]), c(tv[b, h]))
        print(f" rows {r0}..{r0 + 128} of (b={b}, h={h})", flush=True)
        check(oracle, "o", o[b, h, rows], o_ref)
        check(oracle, "to", to[b, h, rows], to_ref)
        check(oracle, "o (forward only)", o_f[b, h, rows], o_ref)
        assert oracle.error_metrics(lse[b, h, rows].cpu(), lse_ref)[0] <= LSE_ABS
        assert oracle.error_metrics(lse_f[b, h, rows].cpu(), lse_ref)[0] <= LSE_ABS


def test_config3_shape_2b_720p_fwd_jvp(pkg, oracle, gpu):
    """The 2B 720p forward + JVP configuration at its real sequence length (L=84480, d=128, bf16, primals N(0,1), tangents N(0,1)*0.1) on 2 of
    the 16 heads (heads are independent; the full-H run is bench.py's), plus properties that need no oracle."""
    (q, k, v, tq, tk, tv), (o, to, lse) = sampled_rows_check(pkg, oracle, gpu, H=2, Lq=84480, Lkv=84480, tangents="full", rms=False)
    dq, dk, dv, dtq, dtk, dtv = (x.to(gpu) for x in (q, k, v, tq, tk, tv))
    # run-to-run reproducibility (fixed sweep order, no atomics)
    o2, to2, lse2 = pkg.fwd_jvp(dq, dk, dv, dtq, dtk, dtv)
    assert torch.equal(o, o2) and torch.equal(to, to2) and torch.equal(lse, lse2)
    # dQ = dK = 0  =>  dO = attention(Q, K, dV): the tangent path reduces to the forward kernel (which walks the keys
    # 64 at a time instead of 32, so the two differ by rounding, not bit for bit)
    _, to_v, _ = pkg.fwd_jvp(dq, dk, dv, torch.zeros_like(dq), torch.zeros_like(dk), dtv)
    o_dv, _, _ = pkg.fwd_jvp(dq, dk, dtv)
    ma, rl = oracle.error_metrics(to_v.float().cpu()[:, :, ::97], o_dv.float().cpu()[:, :, ::97])
    print(f" dV-only tangent vs forward of dV: max_abs={ma:.3e} rel_l2={rl:.3e}", flush=True)
    assert ma <= MAX_ABS and rl <= REL_L2
    # linearity: the q, (k, v) parts of the tangent add up
    _, to_q, _ = pkg.fwd_jvp(dq, dk, dv, dtq)
    _, to_kv, _ = pkg.fwd_jvp(dq, dk, dv, torch.zeros_like(dq), dtk, dtv)
    ma, rl = oracle.error_metrics((to_q.float() + to_kv.float()).cpu()[:, :, ::97], to.float().cpu()[:, :, ::97])
    print(f" linearity: max_abs={ma:.3e} rel_l2={rl:.3e}", flush=True)
    assert ma <= MAX_ABS and rl <= 2 * REL_L2      # three bf16 roundings instead of one
    # forward-only entry returns the same O and LSE up to rounding (it walks the keys 64 at a time)
    o3, none, lse3 = pkg.fwd_jvp(dq, dk, dv)
    assert none is None
    ma, rl = oracle.error_metrics(o3.float().cpu()[:, :, ::97], o.float().cpu()[:, :, ::97])
    print(f" forward-only O vs forward+JVP O: max_abs={ma:.3e} rel_l2={rl:.3e}", flush=True)
    assert ma <= MAX_ABS and rl <= REL_L2
    assert (lse3 - lse).abs().max().item() <= LSE_ABS


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_config1_shape_plumbing_inputs(pkg, oracle, gpu, seed, dtype):
    """The CPU plumbing configuration (B=1, H=16, L=2048, d=128, six fp32 tensors ~N(0,1)*0.5, scale 1/sqrt(128), no
    mask) on the HIP path: the kernels take 16-bit inputs, so the fp32 tensors are rounded to the 16-bit type first.
    Two bars: against torch math SDPA under torch.func.jvp in fp32 on the SAME rounded inputs (the kernel's own error), and
    against it on the ORIGINAL fp32 inputs (kernel error + the rounding of the inputs), both at the 16-bit tolerance."""
    q, k, v, tq, tk, tv = oracle.make_inputs((1, 16, 2048, 128), seed=seed, primal_std=0.5, tangent_std=0.5, dtype=torch.float32)
    half = [x.to(dtype) for x in (q, k, v, tq, tk, tv)]
    o, to, lse = pkg.attention_with_lse(*(x.to(gpu) for x in half))
    torch.cuda.synchronize()
    o_ref, to_ref = oracle.sdpa_jvp_torch(*(x.float() for x in half))
    _, _, lse_ref = oracle.closed_form(*(x.float() for x in half))
    check(oracle, "o (rounded inputs)", o, o_ref)
    check(oracle, "to (rounded inputs)", to, to_ref)
    assert oracle.error_metrics(lse.cpu(), lse_ref)[0] <= LSE_ABS
    o32, to32 = oracle.sdpa_jvp_torch(q, k, v, tq, tk, tv)
    check(oracle, "o (fp32 inputs)", o, o32)
    check(oracle, "to (fp32 inputs)", to, to32)


def test_config2_shape_480p_forward_ragged(pkg, oracle, gpu):
    """The 2B 480p forward-only configuration: L=37440 (not a multiple of 128 or 64), forward only, RMS-normed q/k, LSE returned."""
    sampled_rows_check(pkg, oracle, gpu, H=2, Lq=37440, Lkv=37440, tangents="none", rms=True, seed=1)


def test_config4_shape_14b_rms_normed(pkg, oracle, gpu):
    """The 14B configuration differs from the 2B 720p one in H=40 and RMS-normed q/k: 3 heads at L=84480."""
    sampled_rows_check(pkg, oracle, gpu, H=3, Lq=84480, Lkv=84480, tangents="full", rms=True, seed=2, n_blocks=4)


@pytest.mark.parametrize("tangents", ["q", "none"])
def test_config5_all_heads_takes_the_streaming_kernel(pkg, oracle, gpu, tangents):
    """Configuration 5 with all 16 heads and both batch rows (9376 (query block, head) pairs): the launch the library itself
    sends to the query-streaming kernel, no override; 16 sampled row blocks over heads and batch rows; and bitwise the same
    result from the kernel with one workgroup per query block is not expected (another tile order), only the oracle."""
    g = torch.Generator().manual_seed(1)
    lens = [int(x) for x in torch.randint(64, 513, (2,), generator=g)]
    sampled_rows_check(pkg, oracle, gpu, H=16, Lq=37440, Lkv=512, tangents=tangents, rms=False, key_lens=lens, B=2, seed=4, n_blocks=16)


def test_network_shaped_cross_attention_takes_the_streaming_kernel(pkg, oracle, gpu):
    """The cross-attention call inside the 2B DiT at 720p: B=1, H=16, Lq=84480, Lkv=512, no padding mask, tangent on q."""
    sampled_rows_check(pkg, oracle, gpu, H=16, Lq=84480, Lkv=512, tangents="q", rms=False, B=1, seed=5, n_blocks=8)


def test_config5_shape_cross_attention_key_padding(pkg, oracle, gpu):
    """The text cross-attention configuration: B=2, Lq=37440, Lkv=512, per-row key lengths in 64..512, tangent on q only."""
    g = torch.Generator().manual_seed(0)
    lens = [int(x) for x in torch.randint(64, 513, (2,), generator=g)]
    (q, k, v, tq, _, _), (o, to, lse) = sampled_rows_check(pkg, oracle, gpu, H=4, Lq=37440, Lkv=512, tangents="q", rms=False, key_lens=lens, B=2, seed=3)
    # masked == sliced: row b against only its valid keys, unmasked, must agree bit for bit when the length is a tile multiple
    b = 0
    n = (lens[b] // 32) * 32
    kl = torch.tensor([n, n], dtype=torch.int32, device=gpu)
    o_m, to_m, _ = pkg.fwd_jvp(q[b:b + 1].to(gpu), k[b:b + 1].to(gpu), v[b:b + 1].to(gpu), tq[b:b + 1].to(gpu), key_lens=kl[:1])
    o_s, to_s, _ = pkg.fwd_jvp(q[b:b + 1].to(gpu), k[b:b + 1, :, :n].to(gpu), v[b:b + 1, :, :n].to(gpu), tq[b:b + 1].to(gpu))
    assert torch.equal(o_m, o_s) and torch.equal(to_m, to_s)


def test_environment_variables_do_not_steer_the_kernels(pkg, oracle, gpu, monkeypatch, stream_override):
    """The choice of kernel is the library's (or the explicit hook's): environment variables of the old test hook's names change
    nothing between two calls of one process."""
    q, k, v, tq, _, _ = oracle.make_inputs((1, 2, 1000, 128), (1, 2, 200, 128), seed=12)
    args = [x.to(gpu) for x in (q, k, v, tq)]
    a = pkg.attention_with_lse(*args)
    monkeypatch.setenv("COSMOS_ATTN_STREAM_CHUNK", "3")
    monkeypatch.setenv("COSMOS_ATTN_STREAM_GROUPS", "40")
    b = pkg.attention_with_lse(*args)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    stream_override(chunk=3)
    c = pkg.attention_with_lse(*args)
    o_ref, to_ref, _ = oracle.closed_form(q, k, v, tq, None, None)
    check(oracle, "o (streamed)", c[0], o_ref)
    check(oracle, "to (streamed)", c[1], to_ref)


@pytest.mark.parametrize("tangent_std", [30.0, 300.0])
@pytest.mark.parametrize("tangents", ["full", "q"])
@pytest.mark.parametrize("Lkv", [160, 1024])
def test_fp16_large_tangents_keep_the_reference_range(pkg, oracle, gpu, stream_override, tangent_std, tangents, Lkv):
    """fp16 rounds H = p dS s to a type whose largest value is 65504.  The reference keeps p <= 1
    (flash_attention_jvp_triton.py:104-114), so |dS s| may reach 6.5e4; the kernels keep that range by using the exact running
    max for fp16 with tangents (the lagging max would let p reach 2^6 and overflow from |dS s| ~ 1e3 on).  Tangents of std 30 and
    300 give |dS s| of about 2e2 and 2e3-1e4 at d = 128; the tolerance is the usual one, relative to the size of the tangent."""
    for streamed in (False, True):
        stream_override(chunk=3 if streamed else 1)
        q, k, v, tq, tk, tv = oracle.make_inputs((1, 2, 700, 128), (1, 2, Lkv, 128), seed=int(tangent_std) + Lkv,
                                                 tangent_std=tangent_std, dtype=torch.float16)
        if tangents == "q":
            tk = tv = None
        ds_max = float(((tq.float() @ k.float().transpose(-1, -2)).abs().max()) * 128 ** -0.5)
        dev = lambda x: None if x is None else x.to(gpu)
        o, to, lse = pkg.attention_with_lse(dev(q), dev(k), dev(v), dev(tq), dev(tk), dev(tv))
        torch.cuda.synchronize()
        o_ref, to_ref, _ = oracle.closed_form(q, k, v, tq, tk, tv)
        check(oracle, "o", o, o_ref)
        assert torch.isfinite(to.float()).all(), "tangent overflowed in fp16"
        ma, rl = oracle.error_metrics(to.float().cpu(), to_ref)
        scale = float(abs(to_ref).max())
        print(f"  streamed={streamed} max|dS s|~{ds_max:.3g} max|to|={scale:.3g}: max_abs={ma:.3e} rel_l2={rl:.3e}", flush=True)
        assert rl <= REL_L2 and ma <= MAX_ABS * max(1.0, scale)
