"""The entry point that allocates nothing (cosmos_attn_fwd_jvp_static: workspace in a static device array of the
library) against cosmos_attn_fwd_jvp with a caller-provided workspace, through the C ABI: bitwise equal results, on two
calls in a row, the second on a smaller problem (the array keeps the first call's contents); sizes beyond the array
are refused."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _desc(L, q, k, v, tq, tk, tv, o, to, lse, key_lens=None):
    D = L.AttnDesc()
    D.abi_version, D.dtype = L.ABI_VERSION, L.DTYPE_BF16
    B, H, Lq, d = q.shape
    D.B, D.H, D.Lq, D.Lkv, D.d_qk, D.d_v, D.causal, D.sm_scale = B, H, Lq, k.shape[2], d, v.shape[3], 0, d ** -0.5
    ptr = lambda x: None if x is None else x.data_ptr()
    D.q, D.k, D.v, D.tq, D.tk, D.tv = ptr(q), ptr(k), ptr(v), ptr(tq), ptr(tk), ptr(tv)
    s3 = lambda x: (ctypes.c_int64 * 3)(x.stride(0), x.stride(1), x.stride(2))
    D.q_stride, D.k_stride, D.v_stride, D.o_stride = s3(q), s3(k), s3(v), s3(o)
    D.o, D.to, D.lse, D.key_lens = ptr(o), ptr(to), ptr(lse), ptr(key_lens)
    return D


def _both_ways(pkg, oracle, gpu, shape_q, shape_kv, tangents, seed, key_lens=None):
    L, lib = pkg._lib, pkg._lib.load_library()
    q, k, v, tq, tk, tv = (x.to(gpu) for x in oracle.make_inputs(shape_q, shape_kv, seed=seed))
    if tangents == "q":
        tk = tv = None
    elif tangents == "none":
        tq = tk = tv = None
    kl = None if key_lens is None else torch.tensor(key_lens, dtype=torch.int32, device=gpu)
    st = torch.cuda.current_stream().cuda_stream
    outs = []
    for static in (False, True):
        o = torch.full_like(q, float("nan"))
        to = None if tq is None else torch.full_like(q, float("nan"))
        lse = torch.full(q.shape[:3], float("nan"), device=gpu)
        D = _desc(L, q, k, v, tq, tk, tv, o, to, lse, kl)
        if static:
            rc = lib.cosmos_attn_fwd_jvp_static(ctypes.byref(D), st)
        else:
            n = lib.cosmos_attn_workspace_bytes(ctypes.byref(D))
            assert 0 < n <= lib.cosmos_attn_static_scratch_bytes()
            ws = torch.empty(n, device=gpu, dtype=torch.uint8)
            rc = lib.cosmos_attn_fwd_jvp(ctypes.byref(D), ws.data_ptr(), n, st)
        assert rc == 0, L.status_string(rc)
        torch.cuda.synchronize()
        outs.append((o, to, lse))
    (o0, to0, lse0), (o1, to1, lse1) = outs
    assert torch.isfinite(o1.float()).all()
    assert torch.equal(o0, o1) and torch.equal(lse0, lse1)
    if to0 is not None:
        assert torch.equal(to0, to1)
    o_ref, to_ref, _ = oracle.closed_form(*(None if x is None else x.cpu() for x in (q, k, v, tq, tk, tv)), key_lens=key_lens)
    ma, rl = oracle.error_metrics(o1.float().cpu(), o_ref)
    assert ma <= 2e-2 and rl <= 5e-3


def test_static_scratch_entry_point_matches_workspace_entry_point(pkg, oracle, gpu):
    # text cross-attention shape (tangent on q, key padding), then a smaller one: the array still holds the first image
    _both_ways(pkg, oracle, gpu, (2, 4, 1500, 128), (2, 4, 512, 128), "q", seed=1, key_lens=[300, 77])
    _both_ways(pkg, oracle, gpu, (1, 2, 200, 128), (1, 2, 70, 128), "q", seed=2)
    # self-attention whose thin last round is cut into key ranges (partial results live in the array too), then smaller
    _both_ways(pkg, oracle, gpu, (1, 2, 4096, 128), (1, 2, 4096, 128), "full", seed=3)
    _both_ways(pkg, oracle, gpu, (1, 2, 300, 128), (1, 2, 300, 128), "full", seed=4)
    _both_ways(pkg, oracle, gpu, (1, 3, 1000, 128), (1, 3, 1000, 128), "none", seed=5)


def test_static_scratch_entry_point_refuses_what_does_not_fit(pkg, oracle, gpu):
    L, lib = pkg._lib, pkg._lib.load_library()
    assert lib.cosmos_attn_static_scratch_bytes() == 64 << 20
    q = torch.zeros(1, 16, 128, 128, device=gpu, dtype=torch.bfloat16)
    kv = torch.zeros(1, 16, 40000, 128, device=gpu, dtype=torch.bfloat16)     # image: 16 heads x 1250 tiles x 32 KB = 640 MB
    o, to, lse = torch.empty_like(q), torch.empty_like(q), torch.empty(1, 16, 128, device=gpu)
    D = _desc(L, q, kv, kv, q, kv, kv, o, to, lse)
    assert lib.cosmos_attn_workspace_bytes(ctypes.byref(D)) > lib.cosmos_attn_static_scratch_bytes()
    rc = lib.cosmos_attn_fwd_jvp_static(ctypes.byref(D), torch.cuda.current_stream().cuda_stream)
    assert rc == L.ST_STATIC_SCRATCH
    assert "static scratch" in L.status_string(rc)
    D.abi_version = 0
    assert lib.cosmos_attn_fwd_jvp_static(ctypes.byref(D), None) == L.ST_BAD_ARG


def test_static_scratch_entry_point_under_graph_capture(pkg, oracle, gpu, stream_override):
    """What the entry point is for: a HIP graph captured around it (no allocation inside the capture: the outputs exist
    already), replayed with new input contents and eager work in between, matches eager calls bit for bit.  The streaming
    kernel is forced so that the capture holds the cross-attention path."""
    stream_override(chunk=3)
    L, lib = pkg._lib, pkg._lib.load_library()
    make = lambda seed: [x.to(gpu) for x in oracle.make_inputs((2, 2, 900, 128), (2, 2, 200, 128), seed=seed)[:4]]
    q, k, v, tq = make(0)
    kl = torch.tensor([200, 90], dtype=torch.int32, device=gpu)
    o, to, lse = torch.empty_like(q), torch.empty_like(q), torch.empty(q.shape[:3], device=gpu)
    D = _desc(L, q, k, v, tq, None, None, o, to, lse, kl)
    assert lib.cosmos_attn_fwd_jvp_static(ctypes.byref(D), torch.cuda.current_stream().cuda_stream) == 0   # eager warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        assert lib.cosmos_attn_fwd_jvp_static(ctypes.byref(D), torch.cuda.current_stream().cuda_stream) == 0
    for seed in (1, 2, 3):
        fresh = make(seed)
        for dst, src in zip((q, k, v, tq), fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        o_e, to_e, lse_e = pkg.fwd_jvp(*fresh, key_lens=kl)   # eager work between replays (its own workspace)
        torch.cuda.synchronize()
        assert torch.equal(o, o_e) and torch.equal(to, to_e) and torch.equal(lse, lse_e), seed
