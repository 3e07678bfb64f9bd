"""Benchmark of the attention forward + JVP hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2|c4|c5|c3b|nr|nrb|blk|dblk|dblkf|net|netf|net14|train|e2e2b|e2e14b] [--no-cpu]

A "step" is one call of the hot path (re-tiling kernel + attention kernel, through the Python host and
the C ABI) over one batch of synthetic tensors that are already resident in HBM.  Default workload: the
configuration the headline metric is quoted on -- 2B DiT self-attention forward + JVP at the 720p shape,
B=1, H=16, L=84480, d=128, bf16.  Prints ONE JSON line.

FLOP accounting is the reference's own (cosmos_predict2/_src/predict2/utils/flash_attention_jvp_triton.py:703-713):
2*B*H*Lq*Lkv*d per matmul, 2 matmuls forward, 6 forward + JVP, 5 backward ("2.0 (bwd) + 0.5 (recompute)").
Workload c3b is the backward pass (dq, dk, dv from dout, with the forward's o and lse) at the c3 shape.
Workload nr is the fused RMSNorm + rotary (+ tangent) kernel on one [1, 84480, 16, 128] tensor: HBM-bound, reported
in GB/s of algorithmic bytes (x, tx read once; y, ty written once; the angle table read once).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

REPO_ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, REPO_ROOT)
import __graft_entry__ as entry  # noqa: E402

# MI355X dense bf16 MFMA peak: 256 CU x 4096 FLOP/clk/CU x 2.4 GHz
PEAK_BF16_TFLOPS = 256 * 4096 * 2.4e9 / 1e12

# HBM-side bytes per launch of the dominant kernel.  NOT measured by this program: each figure is copied from a
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE session of this file (FETCH_SIZE x 2 KiB + WRITE_SIZE x 1 KiB; factors calibrated
# with the 1 GiB copy of --copy-calib) whose summary is the named file; the JSON line carries the file name next to the
# number ("traffic_source").  A workload without a counter run reports null.
MEASURED_TRAFFIC_BYTES = {
    "c3": ((2 * 2.633e7 + 710537) * 1024, "profiles/attn_fwd_jvp_kernel_bf16_d128_workload_c3.txt"),
    "nr": ((2 * 359157 + 676527) * 1024, "profiles/norm_rope_kernel_bf16_d128_workload_nr.txt"),
    "c2": ((2 * 1.770e6 + 1.997e5) * 1024, "profiles/attn_fwd_sym_kernel_bf16_d128_workload_c2.txt"),
    "c5": ((2 * 326847 + 603763) * 1024, "profiles/attn_qstream_kernel_bf16_d128_workload_c5.txt"),
    # 8 groups of 2 heads: dK/dV kernel (FETCH 3.22954e6, WRITE 2.7991e7: the dS tiles) + dQ-from-dS pass (FETCH 1.45919e7, WRITE 4.2262e4)
    "c3b": (8 * (2 * (1.23173e6 + 1.42848e7) + 2.7991e7 + 4.22565e4) * 1024, "profiles/attn_bwd_kernel_bf16_d128_workload_c3b.txt"),
}
_NO_TRAFFIC = (None, None)

WORKLOADS = {
    # name: (description, B, H, Lq, Lkv, d, tangents, rms-normed q/k, key-padding)
    "c2": ("2B DiT self-attention fwd bf16 480p B1 H16 L37440 d128", 1, 16, 37440, 37440, 128, "none", True, False),
    "c3": ("2B DiT self-attention fwd+JVP bf16 720p B1 H16 L84480 d128", 1, 16, 84480, 84480, 128, "full", False, False),
    "c4": ("14B DiT self-attention fwd+JVP bf16 720p B1 H40 L84480 d128", 1, 40, 84480, 84480, 128, "full", True, False),
    "c5": ("2B DiT text cross-attention fwd+JVP bf16 B2 H16 Lq37440 Lkv512 d128 key-padding tangent-on-q", 2, 16, 37440, 512, 128, "q", False, True),
    "c3b": ("2B DiT self-attention backward bf16 720p B1 H16 L84480 d128", 1, 16, 84480, 84480, 128, "bwd", False, False),
    # the step before attention: per-head RMSNorm + rotary embedding of q (or k) with its tangent, one tensor per call
    "nr": ("2B DiT q RMSNorm+RoPE+tangent bf16 720p B1 S84480 H16 d128", 1, 16, 84480, 84480, 128, "norm_rope", False, False),
    "nrb": ("2B DiT q RMSNorm+RoPE backward bf16 720p B1 S84480 H16 d128", 1, 16, 84480, 84480, 128, "norm_rope_bwd", False, False),
    # the whole DiT self-attention module with a tangent: 4 projections (library GEMMs on stacked primal + tangent),
    # RMSNorm + RoPE (+ tangent) of q and k, attention forward + JVP
    "blk": ("2B DiT self-attention module fwd+JVP bf16 720p B1 L84480 K2048 H16 d128", 1, 16, 84480, 84480, 128, "module", False, False),
    # one whole DiT block with a tangent: adaLN modulation, self-attention, text cross-attention, MLP, gated residuals
    "dblkf": ("2B DiT block forward (inference) bf16 720p B1 T24 H44 W80 D2048 heads16 text512x1024 adaLN-LoRA256", 1, 16, 84480, 512, 128, "block_fwd", False, False),
    "dblk": ("2B DiT block fwd+JVP bf16 720p B1 T24 H44 W80 D2048 heads16 text512x1024 adaLN-LoRA256", 1, 16, 84480, 512, 128, "block", False, False),
    # the whole 2B video-conditioned DiT (28 blocks; patch / time embedding, text projection 100352 -> 1024, final layer)
    "netf": ("2B DiT network forward (inference) bf16 720p B1 x16x24x88x160 28 blocks D2048 heads16 text512x100352", 1, 16, 84480, 512, 128, "network_fwd", False, False),
    "net": ("2B DiT network fwd+JVP along (x, t) bf16 720p B1 x16x24x88x160 28 blocks D2048 heads16 text512x100352", 1, 16, 84480, 512, 128, "network", False, False),
    # one training step of the whole 2B network: forward, backward through every block (attention backward kernels, RMSNorm +
    # RoPE backward, library GEMMs), blocks checkpointed (sac_config) so that the activations fit
    "train": ("2B DiT network forward + backward (block-wise activation checkpointing) bf16 720p B1 x16x24x88x160 28 blocks", 1, 16, 84480, 512, 128, "network_train", False, False),
    "net14": ("14B DiT network fwd+JVP along (x, t) bf16 720p B1 x16x24x88x160 36 blocks D5120 heads40 text512x100352", 1, 40, 84480, 512, 128, "network", False, False),
    # the reference's own end-to-end inference timing (networks/minimal_v4_dit_test_sparse_attn_e2e_speedup.py:287-375,
    # dense self-attention cases): text-to-world MiniTrainDIT, x [1,16,24,88,160], text [1,512,1024], forward under no_grad
    "e2e2b": ("2B text2world DiT inference forward bf16 720p B1 x16x24x88x160 28 blocks D2048 heads16 text512x1024", 1, 16, 84480, 512, 128, "e2e", False, False),
    "e2e14b": ("14B text2world DiT inference forward bf16 720p B1 x16x24x88x160 36 blocks D5120 heads40 text512x1024", 1, 40, 84480, 512, 128, "e2e", False, False),
}
PEAK_HBM_GBS = 8000.0


def make_device_inputs(B, H, Lq, Lkv, d, tangents, rms, dev, seed=0):
    """Synthetic tensors generated on the GPU per head block (values ~N(0,1), tangents ~N(0,1)*0.1)."""
    g = torch.Generator(device=dev).manual_seed(seed)

    def rn(L, std, norm=False):
        x = torch.randn((B, H, L, d), generator=g, device=dev, dtype=torch.float32) * std
        if norm:
            x = x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + 1e-6)
        return x.to(torch.bfloat16)

    q, k, v = rn(Lq, 1.0, rms), rn(Lkv, 1.0, rms), rn(Lkv, 1.0)
    tq = rn(Lq, 0.1) if tangents != "none" else None
    tk = rn(Lkv, 0.1) if tangents == "full" else None
    tv = rn(Lkv, 0.1) if tangents == "full" else None
    return q, k, v, tq, tk, tv


def cpu_baseline(oracle, H, Lkv, d, tangents, rows=512, seed=0):
    """The reference's CPU path -- torch math SDPA under torch.func.jvp, fp32 -- timed on this host's cores
    on a bounded sample: `rows` query rows against the full K/V for all heads (query rows are independent,
    so FLOP/s on the sample is FLOP/s of the whole call)."""
    q, k, v, tq, tk, tv = oracle.make_inputs((1, H, rows, d), (1, H, Lkv, d), seed=seed, dtype=torch.float32)
    if tangents == "none":
        fn = lambda: oracle.sdpa_forward_torch(q, k, v)
        n_mm = 2
    else:
        if tangents == "q":
            tk = tv = None
        fn = lambda: oracle.sdpa_jvp_torch(q, k, v, tq, tk, tv)
        n_mm = 6
    fn()  # warm-up
    t0 = time.perf_counter()
    reps = 0
    while True:
        fn()
        reps += 1
        el = time.perf_counter() - t0
        if el > 10.0 or reps >= 5:
            break
    sec = el / reps
    flops = n_mm * 2.0 * H * rows * Lkv * d
    return {
        "value": flops / sec / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "host_cpus": os.cpu_count(),
        "kind": "port",
        "sample": f"torch math SDPA + torch.func.jvp fp32, {rows} query rows x full Lkv={Lkv} x {H} heads, "
                  f"{reps} reps, {sec:.3f} s per rep; rows are independent so the rate extrapolates to the full call",
    }


def rope_angles(pkg, dev, T, Hh, W, D):
    """The rotary angle table [T*Hh*W, D] fp32 of the DiT's positional embedder (the package's own host-side class)."""
    pe = pkg.VideoRopePosition3DEmb(head_dim=D, len_h=Hh, len_w=W, len_t=T, enable_fps_modulation=False).to(dev)
    return pe.generate_embeddings((1, T, Hh, W, D)).reshape(T * Hh * W, D).contiguous()


def gemm_reference(dev):
    """TFLOP/s of torch.matmul (hipBLASLt) on square bf16 operands: context for the roofline fraction."""
    out = {}
    for n, reps in ((8192, 20), (16384, 5)):
        a = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
        b = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
        for _ in range(3):
            c = a @ b
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            c = a @ b
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        out[f"{n}^3"] = {"ms": ms, "tflops": 2.0 * n ** 3 / ms / 1e9}
        del a, b, c
    return out


def bench_backward(args, pkg, dev, desc_txt, B, H, Lq, Lkv, d, steps, warmup):
    """One step = cosmos_attn_bwd (statistics, two stream re-tilings, dK/dV kernel, dQ kernel) through the Python host."""
    q, k, v, dout, _, _ = make_device_inputs(B, H, Lq, Lkv, d, "q", False, dev)
    dout = dout * 10.0   # ~N(0, 1)
    o, _, lse = pkg.fwd_jvp(q, k, v)
    flops = 5 * 2.0 * B * H * Lq * Lkv * d   # the reference's accounting: 5 matmuls
    step = lambda: pkg.bwd(q, k, v, o, lse, dout)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        out = step()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / steps
    del out
    ms = []
    for i in range(steps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(); out = step(); e1.record()
        torch.cuda.synchronize()
        ms.append(e0.elapsed_time(e1))
        del out
    avg = sum(ms) / len(ms)
    achieved = flops / (avg * 1e-3) / 1e12
    parity = backward_sampled_parity(entry.load_oracle(), (q, k, v, o, lse, dout), step())
    result = {
        "parity_sampled": parity,
        "metric": "attn backward TFLOP/s & % bf16 MFMA peak @ 2B 720p (L=84480); ms per call",
        "value": flops / sec / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": desc_txt, "B": B, "H": H, "Lq": Lq, "Lkv": Lkv, "d": d, "flop_per_call": flops,
                   "executed_matmuls": 5, "pct_of_bf16_mfma_peak": 100.0 * flops / sec / 1e12 / PEAK_BF16_TFLOPS},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS, "traffic": MEASURED_TRAFFIC_BYTES["c3b"][0], "traffic_source": MEASURED_TRAFFIC_BYTES["c3b"][1],
                     "kernel": "cosmos_attn_bwd (per group of heads: attn_dkdv_quad_kernel keeping dS, attn_dq_from_ds_kernel; 3 small launches)", "kernel_ms_avg": avg, "kernel_ms_min": min(ms)},
    }
    return result


def backward_sampled_parity(oracle, inputs, grads, n_blocks=4, seed=0):
    """Sampled 128-row blocks of dq and 128-key blocks of dk, dv (first, last, random; heads drawn over all of them) of one
    backward call against the fp32 row / key block oracles on the CPU, outside the timed region.  Tolerance of the backward
    tests: relative-L2 <= 1e-2 and max-abs <= 2e-2 * max(1, max|want|) per block."""
    import numpy as np

    q, k, v, o, lse, dout = inputs
    dq, dk, dv = grads
    B, H, Lq, _ = q.shape
    Lkv = k.shape[2]
    rng = np.random.default_rng(seed)
    worst = {"rel_l2": 0.0, "max_abs_over_limit": 0.0}

    def fold(got, want):
        ma, rl = oracle.error_metrics(got.float().cpu(), want)
        worst["rel_l2"] = max(worst["rel_l2"], rl)
        worst["max_abs_over_limit"] = max(worst["max_abs_over_limit"], ma / (2e-2 * max(1.0, float(want.abs().max()))))

    c = lambda x: x.cpu()
    for i in range(n_blocks):
        b, h = i % B, int(rng.integers(0, H))
        r0 = [0, max(Lq - 128, 0)][i] if i < 2 else int(rng.integers(0, max(Lq - 128, 1)))
        rows = slice(r0, min(r0 + 128, Lq))
        fold(dq[b, h, rows], oracle.grads_rows_oracle(c(q[b, h, rows]), c(k[b, h]), c(v[b, h]), c(dout[b, h, rows])))
        c0 = [max(Lkv - 128, 0), 0][i] if i < 2 else int(rng.integers(0, max(Lkv - 128, 1)))
        cols = slice(c0, min(c0 + 128, Lkv))
        wk, wv = oracle.grads_cols_oracle(c(q[b, h]), c(k[b, h, cols]), c(v[b, h, cols]), c(o[b, h]), c(lse[b, h]), c(dout[b, h]))
        fold(dk[b, h, cols], wk)
        fold(dv[b, h, cols], wv)
    worst["blocks"] = n_blocks
    worst["rows_per_block"] = 128
    worst["within_tolerance"] = bool(worst["rel_l2"] <= 1e-2 and worst["max_abs_over_limit"] <= 1.0)
    return worst


def bench_module(args, pkg, dev, desc_txt, B, H, L, D):
    """One step = Attention.forward_jvp(x, tx, rope_emb) of the 2B DiT's self-attention module (K = H * D)."""
    K = H * D
    torch.manual_seed(0)
    m = pkg.Attention(K, None, n_heads=H, head_dim=D)
    m.init_weights()
    m = m.to(device=dev, dtype=torch.bfloat16).eval()
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn((B, L, K), generator=g, device=dev).to(torch.bfloat16)
    tx = (torch.randn((B, L, K), generator=g, device=dev) * 0.1).to(torch.bfloat16)
    rope = rope_angles(pkg, dev, 24, 44, 80, D).reshape(L, 1, 1, D)
    flops_gemm = 4 * 2 * 2.0 * B * L * K * K              # q, k, v, output projections on primal and tangent
    flops_attn = 6 * 2.0 * B * H * L * L * D
    flops = flops_gemm + flops_attn
    step = lambda: m.forward_jvp(x, tx, rope_emb=rope)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        out = step()
    e1.record()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / args.steps
    avg = e0.elapsed_time(e1) / args.steps
    del out
    achieved = flops / (avg * 1e-3) / 1e12
    result = {
        "metric": "DiT self-attention module fwd+JVP TFLOP/s & % bf16 MFMA peak @ 2B 720p (L=84480); ms per call",
        "value": flops / sec / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": desc_txt, "B": B, "L": L, "K": K, "H": H, "d": D, "flop_per_call": flops,
                   "flop_gemm": flops_gemm, "flop_attention": flops_attn,
                   "pct_of_bf16_mfma_peak": 100.0 * flops / sec / 1e12 / PEAK_BF16_TFLOPS},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS, "traffic": None,
                     "kernel": "whole module call (attn_fwd_jvp_kernel dominates)", "kernel_ms_avg": avg},
    }
    print(json.dumps(result), flush=True)


def bench_block(args, pkg, dev, desc_txt, B, H, L, Mk, D, forward_only=False):
    """One step = Block.forward_jvp (or, with ``forward_only``, Block.forward under no_grad) of the 2B DiT's transformer
    block at the 720p token grid."""
    K, Kc, T, Hh, W = H * D, 1024, 24, 44, 80
    assert T * Hh * W == L
    torch.manual_seed(0)
    m = pkg.Block(K, Kc, H, mlp_ratio=4.0, use_adaln_lora=True, adaln_lora_dim=256)
    m.init_weights()
    with torch.no_grad():   # a freshly initialised block has zero gates; give the modulation something to do
        for mod in (m.adaln_modulation_self_attn, m.adaln_modulation_cross_attn, m.adaln_modulation_mlp):
            mod[-1].weight.copy_(torch.randn_like(mod[-1].weight) / 16.0)
    m = m.to(device=dev, dtype=torch.bfloat16).eval()
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(s, generator=g, device=dev)
    x, tx = rn(B, T, Hh, W, K).bfloat16(), (0.1 * rn(B, T, Hh, W, K)).bfloat16()
    emb, temb = rn(B, T, K).bfloat16(), (0.1 * rn(B, T, K)).bfloat16()
    lora, tlora = (0.3 * rn(B, T, 3 * K)).bfloat16(), (0.03 * rn(B, T, 3 * K)).bfloat16()
    ctx = rn(B, Mk, Kc).bfloat16()
    rope = rope_angles(pkg, dev, T, Hh, W, D).reshape(L, 1, 1, D)
    gemm = lambda rows, k, n: 2.0 * rows * k * n
    flops = {
        "self_attn_projections": 4 * 2 * gemm(B * L, K, K),
        "self_attn": 6 * 2.0 * B * H * L * L * D,
        "cross_attn_projections": 2 * 2 * gemm(B * L, K, K) + 2 * gemm(B * Mk, Kc, K),
        "cross_attn": 4 * 2.0 * B * H * L * Mk * D,
        "mlp": 2 * 2 * gemm(B * L, K, 4 * K),
    }
    step = lambda: m.forward_jvp(x, tx, emb, temb, ctx, rope, lora, tlora)
    if forward_only:     # no tangents: half the GEMM work, 2 attention matmuls instead of 6 (4)
        flops = {k: v / 2 for k, v in flops.items()}
        flops["self_attn"] = 2 * 2.0 * B * H * L * L * D
        flops["cross_attn"] = 2 * 2.0 * B * H * L * Mk * D
        flops["cross_attn_projections"] = 2 * gemm(B * L, K, K) + 2 * gemm(B * Mk, Kc, K)

        def step():
            with torch.no_grad():
                return m(x, emb, ctx, rope, lora)
    total = sum(flops.values())
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        out = step()
    e1.record()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / args.steps
    avg = e0.elapsed_time(e1) / args.steps
    del out
    achieved = total / (avg * 1e-3) / 1e12
    result = {
        "metric": ("DiT block forward" if forward_only else "DiT block fwd+JVP") + " TFLOP/s & % bf16 MFMA peak @ 2B 720p (L=84480); ms per call",
        "value": total / sec / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": desc_txt, "flop_per_call": total, "flop_parts": flops,
                   "pct_of_bf16_mfma_peak": 100.0 * total / sec / 1e12 / PEAK_BF16_TFLOPS},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS, "traffic": None,
                     "kernel": "whole block call (the attention kernel dominates)", "kernel_ms_avg": avg},
    }
    print(json.dumps(result), flush=True)


def bench_network(args, pkg, dev, desc_txt, B, H, L, Mk, D, forward_only=False, text2world=False, train=False):
    """One step = MinimalV1LVGDiT.forward_jvp (or, with ``forward_only``, its forward under no_grad) of the 2B DiT:
    16 latent channels x 24 latent frames x 88 x 160, 2 x 2 patches -> 84480 tokens, 28 blocks.  ``text2world``: the
    plain MiniTrainDIT of the reference's end-to-end timing script (no condition mask, text context already 1024 wide;
    36 blocks when H = 40)."""
    K, Kc, Kin, T, Hh, W, C, n_blocks = H * D, 1024, 100352, 24, 88, 160, 16, (36 if H == 40 else 28)
    assert T * (Hh // 2) * (W // 2) == L
    torch.manual_seed(0)
    common = dict(max_img_h=240, max_img_w=240, max_frames=128, in_channels=C, out_channels=C, patch_spatial=2, patch_temporal=1,
                  model_channels=K, num_blocks=n_blocks, num_heads=H, concat_padding_mask=True, use_adaln_lora=True,
                  adaln_lora_dim=256, crossattn_emb_channels=Kc)
    with torch.device(dev):
        torch.set_default_dtype(torch.bfloat16)     # 14B parameters: initialise them in 16 bits on the device
        try:
            if text2world:
                net = pkg.MiniTrainDIT(**common)
                Kin = Kc
            else:
                # the released 2B rectified-flow configuration: text projection 100352 -> 1024, fp32 time embedding /
                # modulation / final layer (configs/video2world/experiment/reason_embeddings/model_2B_reason_1p1_rectified_flow.py:321-324)
                net = pkg.MinimalV1LVGDiT(use_crossattn_projection=True, crossattn_proj_in_channels=Kin,
                                          use_wan_fp32_strategy=True, sac_config=dict(mode="block_wise") if train else None, **common)
        finally:
            torch.set_default_dtype(torch.float32)
        with torch.no_grad():   # a freshly initialised network has zero modulation layers; give them something to do
            for blk in net.blocks:
                for mod in (blk.adaln_modulation_self_attn, blk.adaln_modulation_cross_attn, blk.adaln_modulation_mlp):
                    mod[-1].weight.copy_(torch.randn_like(mod[-1].weight) / 64.0)
            net.final_layer.adaln_modulation[-1].weight.copy_(torch.randn_like(net.final_layer.adaln_modulation[-1].weight) / 16.0)
    net = net.to(dtype=torch.bfloat16)
    net = net.train() if train else net.eval()
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(s, generator=g, device=dev)
    x, tx = rn(B, C, T, Hh, W).bfloat16(), (0.1 * rn(B, C, T, Hh, W)).bfloat16()
    t_dtype = torch.bfloat16 if text2world else torch.float32      # fp32 timesteps with the fp32 strategy
    ts = torch.full((B, 1), 0.6, device=dev, dtype=t_dtype)
    tts = torch.full((B, 1), 0.5, device=dev, dtype=t_dtype)
    ctx = rn(B, Mk, Kin).bfloat16()
    cond = torch.zeros(B, 1, T, Hh, W, device=dev, dtype=torch.bfloat16)
    cond[:, :, :1] = 1
    pm = torch.zeros(B, 1, Hh, W, device=dev, dtype=torch.bfloat16)
    fps = torch.full((B,), 16.0, device=dev)
    gemm = lambda rows, k, n: 2.0 * rows * k * n
    cin = (C + (1 if text2world else 2)) * 4
    per_block = (4 * 2 * gemm(B * L, K, K) + 6 * 2.0 * B * H * L * L * D + 2 * 2 * gemm(B * L, K, K) + 2 * gemm(B * Mk, Kc, K)
                 + 4 * 2.0 * B * H * L * Mk * D + 2 * 2 * gemm(B * L, K, 4 * K))
    ends = 2 * gemm(B * L, cin, K) + 2 * gemm(B * L, K, 4 * C) + gemm(B * Mk, Kin, Kc)
    step = lambda: net.forward_jvp(x, tx, ts, tts, ctx, cond, fps=fps, padding_mask=pm)
    if text2world:
        assert forward_only
    if train:
        # model FLOP of a training step: GEMMs 3 x forward (forward, grad of input, grad of weight), attention 1 + 2.5 x forward
        # (5 matmuls backward for 2 forward); the recomputed forward of the checkpointed blocks is not counted
        gemm_f = 4 * gemm(B * L, K, K) + 2 * gemm(B * L, K, K) + 2 * gemm(B * Mk, Kc, K) + 2 * gemm(B * L, K, 4 * K)
        attn_f = 2 * 2.0 * B * H * L * L * D + 2 * 2.0 * B * H * L * Mk * D
        per_block = 3 * gemm_f + 3.5 * attn_f
        ends = 3 * (gemm(B * L, cin, K) + gemm(B * L, K, 4 * C) + gemm(B * Mk, Kin, Kc))
        params = [p_ for p_ in net.parameters() if p_.requires_grad]

        def step():
            for p_ in params:
                p_.grad = None
            out_ = net(x, ts, ctx, cond, fps=fps, padding_mask=pm)
            out_.float().square().mean().backward()
            return out_.detach()
    elif forward_only:
        per_block = (4 * gemm(B * L, K, K) + 2 * 2.0 * B * H * L * L * D + 2 * gemm(B * L, K, K) + 2 * gemm(B * Mk, Kc, K)
                     + 2 * 2.0 * B * H * L * Mk * D + 2 * gemm(B * L, K, 4 * K))
        ends = gemm(B * L, cin, K) + gemm(B * L, K, 4 * C) + (0 if text2world else gemm(B * Mk, Kin, Kc))

        def step():
            with torch.no_grad():
                if text2world:
                    return net(x, ts, ctx, fps=fps, padding_mask=pm)
                return net(x, ts, ctx, cond, fps=fps, padding_mask=pm)
    total = n_blocks * per_block + ends
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        out = step()
    e1.record()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / args.steps
    avg = e0.elapsed_time(e1) / args.steps
    del out
    achieved = total / (avg * 1e-3) / 1e12
    result = {
        "metric": ("DiT network forward + backward" if train else "DiT network forward" if forward_only else "DiT network fwd+JVP") + f" TFLOP/s & % bf16 MFMA peak @ 720p (L=84480, {n_blocks} blocks of {K}); ms per call",
        "value": total / sec / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": desc_txt, "flop_per_call": total, "flop_per_block": per_block, "flop_outside_blocks": ends,
                   "peak_memory_gb": torch.cuda.max_memory_allocated() / 1e9,
                   "pct_of_bf16_mfma_peak": 100.0 * total / sec / 1e12 / PEAK_BF16_TFLOPS},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS, "traffic": None,
                     "kernel": "whole network call (the attention kernel dominates)", "kernel_ms_avg": avg},
    }
    print(json.dumps(result), flush=True)


def copy_calibration(dev):
    """One plain elementwise copy kernel that reads 1 GiB and writes 1 GiB: the known-size launch the FETCH_SIZE /
    WRITE_SIZE counters are scaled by."""
    src = torch.empty(1 << 30, device=dev, dtype=torch.uint8).fill_(1)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


def bench_norm_rope(args, pkg, dev, desc_txt, B, H, S, D, backward=False):
    """One step = cosmos_norm_rope on x, tx [B, S, H, D] bf16 -> y, ty (heads-first), through the Python host; with
    ``backward`` one step = cosmos_norm_rope_bwd on x, dy -> dx, dweight (x, dy read once, dx written once)."""
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn((B, S, H, D), generator=g, device=dev).to(torch.bfloat16)
    tx = (torch.randn((B, S, H, D), generator=g, device=dev) * 0.1).to(torch.bfloat16)
    w = (1.0 + 0.1 * torch.randn(D, generator=g, device=dev)).float()
    angles = rope_angles(pkg, dev, 24, 44, 80, D)   # 24 x 44 x 80 = 84480 tokens
    assert angles.shape[0] == S
    nbytes = 4 * x.numel() * 2 + angles.numel() * 4 + D * 4     # x, tx in; y, ty out; angles; weight
    step = lambda: pkg.norm_rope(x, w, angles, tx, out_layout="bhsd")
    if backward:
        dy = tx.transpose(1, 2).contiguous().transpose(1, 2)       # the gradient arrives in heads-first memory
        nbytes = 3 * x.numel() * 2 + angles.numel() * 4 + D * 4   # x, dy in; dx out; angles; weight (partial sums: 2.7 MB)
        step = lambda: pkg.norm_rope_bwd(x, w, angles, dy)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # one launch per step: HIP events on the launch stream around the timed region give the average launch duration
    # (events around a single 0.3 ms launch would mostly time the host getting to the launch)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        out = step()
    e1.record()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / args.steps
    avg = e0.elapsed_time(e1) / args.steps
    achieved = nbytes / (avg * 1e-3) / 1e9
    result = {
        "metric": ("q/k RMSNorm+RoPE backward" if backward else "q/k RMSNorm+RoPE+tangent") +
                  " GB/s of algorithmic bytes @ 2B 720p (S=84480, H=16, d=128); ms per call",
        "value": nbytes / sec / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": desc_txt, "B": B, "S": S, "H": H, "D": D, "bytes_per_call": nbytes},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": achieved / PEAK_HBM_GBS, "traffic": None if backward else MEASURED_TRAFFIC_BYTES["nr"][0], "traffic_source": None if backward else MEASURED_TRAFFIC_BYTES["nr"][1],
                     "kernel": "norm_rope_bwd_kernel<16, bf16> + norm_rope_dweight_kernel" if backward else "norm_rope_kernel<16, tangent, bf16>",
                     "kernel_ms_avg": avg},
    }
    if args.copy_calib:
        copy_calibration(dev)
    if not args.no_cpu and not backward:
        # the same step in torch fp32 on the host cores (library rms_norm + rotation under forward AD), on a sample
        nro = entry.load_norm_rope_oracle()
        rows = 2048
        xs, txs, ws, as_ = x[:, :rows].float().cpu(), tx[:, :rows].float().cpu(), w.cpu().numpy(), angles[:rows].cpu().numpy()
        nro.norm_rope_torch(xs, ws, as_, txs)
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < 5.0 and reps < 20:
            nro.norm_rope_torch(xs, ws, as_, txs)
            reps += 1
        csec = (time.perf_counter() - t0) / reps
        cbytes = 4 * xs.numel() * 2 + as_.size * 4
        result["cpu_baseline"] = {"value": cbytes / csec / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                                  "sample": f"torch rms_norm + rotate-half under torch.func.jvp fp32, first {rows} positions x {H} heads, "
                                            f"{reps} reps, {csec:.4f} s per rep; same 16-bit byte accounting as the GPU figure"}
    print(json.dumps(result), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="headline workload only: skip the short timings of c2, c4, c5, c3b")
    ap.add_argument("--extra-steps", type=int, default=5, help="timed steps of each of the extra workloads")
    ap.add_argument("--gemm-ref", action="store_true",
                    help="also time the vendor bf16 GEMM (torch.matmul) at 8192^3 and 16384^3: what dense MFMA work sustains on this box")
    ap.add_argument("--copy-calib", action="store_true",
                    help="also run one plain 1 GiB device copy (calibrates FETCH_SIZE / WRITE_SIZE counters under rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the hot path is a single-GPU kernel; "
              "sharding across GPUs is design-only). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    pkg = entry.load_package()
    lib = pkg._lib.load_library()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    desc_txt, B, H, Lq, Lkv, d, tangents, rms, padded = WORKLOADS[args.workload]
    if tangents == "bwd":
        result = bench_backward(args, pkg, dev, desc_txt, B, H, Lq, Lkv, d, steps=args.steps, warmup=args.warmup)
        if args.copy_calib:
            copy_calibration(dev)
        print(json.dumps(result), flush=True)
        return
    if tangents == "e2e":
        return bench_network(args, pkg, dev, desc_txt, B, H, Lq, Lkv, d, forward_only=True, text2world=True)
    if tangents == "network_train":
        return bench_network(args, pkg, dev, desc_txt, B, H, Lq, Lkv, d, train=True)
    if tangents in ("network", "network_fwd"):
        return bench_network(args, pkg, dev, desc_txt, B, H, Lq, Lkv, d, forward_only=tangents == "network_fwd")
    if tangents in ("block", "block_fwd"):
        return bench_block(args, pkg, dev, desc_txt, B, H, Lq, Lkv, d, forward_only=tangents == "block_fwd")
    if tangents == "module":
        return bench_module(args, pkg, dev, desc_txt, B, H, Lq, d)
    if tangents in ("norm_rope", "norm_rope_bwd"):
        return bench_norm_rope(args, pkg, dev, desc_txt, B, H, Lq, d, backward=tangents == "norm_rope_bwd")
    result = bench_attention(args, pkg, lib, dev, args.workload, args.steps, args.warmup, full=True)
    if args.workload == "c3" and not args.no_extra:
        # the other configurations of the hot path under the same clock, a few steps each (the headline fields above
        # are not touched): name -> ms per call through the Python host, TFLOP/s and fraction of the bf16 MFMA peak
        # by the algorithmic FLOP count, the dominant kernel alone
        extra = {}
        for name in ("c2", "c4", "c5", "c3b"):
            torch.cuda.empty_cache()
            if WORKLOADS[name][6] == "bwd":
                r = bench_backward(args, pkg, dev, *WORKLOADS[name][:6], steps=args.extra_steps, warmup=2)
                r["config"]["workload"] = WORKLOADS[name][0]
            else:
                # (the sub-millisecond call gets ten times the steps: five of them are over before the clock has settled)
                short = name == "c5"
                r = bench_attention(args, pkg, lib, dev, name, args.extra_steps * (10 if short else 1), 10 if short else 2, full=False)
            extra[name] = {"workload": r["config"]["workload"], "ms": r["ms_per_step"], "tflops": r["value"],
                           "frac": r["value"] / PEAK_BF16_TFLOPS, "kernel_ms": r["roofline"]["kernel_ms_avg"],
                           "roofline_bound": r["roofline"]["bound"], "roofline_frac": r["roofline"]["frac"], "steps": r["steps"],
                           "parity_sampled": r["parity_sampled"], "within_tolerance": r["parity_sampled"]["within_tolerance"]}
            if "ms_per_step_one_call" in r:
                extra[name]["ms_one_call"] = r["ms_per_step_one_call"]
        result["extra"] = extra
    print(json.dumps(result), flush=True)


def sampled_parity(oracle, tensors, outputs, key_lens, n_blocks=6, seed=0):
    """128-row blocks (first, last, random; heads drawn over all of them) of the outputs of a call against the fp32 row-block
    oracle on the CPU.  Returns the largest max-abs / relative-L2 errors over the blocks (O and dO) and the LSE error."""
    import numpy as np

    q, k, v, tq, tk, tv = tensors
    o, to, lse = outputs
    B, H, Lq, _ = q.shape
    rng = np.random.default_rng(seed)
    starts = [0, max(Lq - 128, 0)] + [int(x) for x in rng.integers(0, max(Lq - 128, 1), n_blocks - 2)]
    worst = {"max_abs": 0.0, "rel_l2": 0.0, "lse_max_abs": 0.0}
    c = lambda x: None if x is None else x.cpu()
    for i, r0 in enumerate(starts):
        b, h = i % B, int(rng.integers(0, H))
        rows = slice(r0, min(r0 + 128, Lq))
        o_ref, to_ref, lse_ref = oracle.rows_oracle(c(q[b, h, rows]), c(k[b, h]), c(v[b, h]), None if tq is None else c(tq[b, h, rows]),
                                                    None if tk is None else c(tk[b, h]), None if tv is None else c(tv[b, h]),
                                                    kv_len=None if key_lens is None else int(key_lens[b]))
        for got, want in ((o, o_ref), (to, to_ref)):
            if got is None:
                continue
            ma, rl = oracle.error_metrics(got[b, h, rows].float().cpu(), want)
            worst["max_abs"], worst["rel_l2"] = max(worst["max_abs"], ma), max(worst["rel_l2"], rl)
        worst["lse_max_abs"] = max(worst["lse_max_abs"], oracle.error_metrics(lse[b, h, rows].cpu(), lse_ref)[0])
    worst["blocks"] = len(starts)
    worst["rows_per_block"] = 128
    worst["within_tolerance"] = bool(worst["max_abs"] <= 2e-2 and worst["rel_l2"] <= 5e-3 and worst["lse_max_abs"] <= 2e-3)
    return worst


def bench_attention(args, pkg, lib, dev, name, steps, warmup, full=True):
    """One step = pkg.fwd_jvp (re-tiling kernel + attention kernel through the Python host and the C ABI).  ``full``:
    also the CPU baseline, the parity check of the timed call's own output and the optional calibration legs."""
    desc_txt, B, H, Lq, Lkv, d, tangents, rms, padded = WORKLOADS[name]
    q, k, v, tq, tk, tv = make_device_inputs(B, H, Lq, Lkv, d, tangents, rms, dev)
    key_lens = None
    mean_len = Lkv
    if padded:
        g = torch.Generator().manual_seed(0)
        kl = torch.randint(64, Lkv + 1, (B,), generator=g)
        key_lens = kl.to(device=dev, dtype=torch.int32)
        mean_len = float(kl.float().mean())
    n_mm = 2 if tangents == "none" else 6
    flops = n_mm * 2.0 * B * H * Lq * Lkv * d            # nominal (padded Lkv), the reference's accounting
    n_mm_alg = {"none": 2, "q": 4, "full": 6}[tangents]  # matmuls that are not identically zero
    flops_alg = n_mm_alg * 2.0 * B * H * Lq * mean_len * d

    def one_call():
        return pkg.fwd_jvp(q, k, v, tq, tk, tv, key_lens=key_lens)

    def timed(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            out = fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps, out

    sec_one_call = None
    if padded:
        # Text cross-attention: the context's keys / values are the same for every block call and every sampling step, so the
        # module mirror re-tiles them once (pack_kv) and runs against the image (run_packed).  That is the step timed here; the
        # one-call form (re-tiling + allocation inside every call) is reported beside it.
        sec_one_call, _ = timed(one_call)
        packed = pkg.pack_kv(k, v)
        step = lambda: pkg.run_packed(q, packed, tq, key_lens=key_lens)
    else:
        step = one_call
    sec, out_timed = timed(step)          # the last timed step's output is kept for the parity check after all timing

    # dominant kernel alone (the attention kernel and its few-microsecond merge kernel), HIP events on the launch stream
    import ctypes
    from types import SimpleNamespace

    o = torch.empty((B, H, Lq, d), device=dev, dtype=torch.bfloat16)
    to = torch.empty_like(o) if tangents != "none" else None
    lse = torch.empty((B, H, Lq), device=dev, dtype=torch.float32)
    D = pkg._lib.AttnDesc()
    D.abi_version, D.dtype = pkg._lib.ABI_VERSION, pkg._lib.DTYPE_BF16
    D.B, D.H, D.Lq, D.Lkv, D.d_qk, D.d_v, D.causal, D.sm_scale = B, H, Lq, Lkv, d, d, 0, d ** -0.5
    ptr = lambda x: None if x is None else x.data_ptr()
    D.q, D.k, D.v, D.tq, D.tk, D.tv = ptr(q), ptr(k), ptr(v), ptr(tq), ptr(tk), ptr(tv)
    s3 = lambda x: (ctypes.c_int64 * 3)(x.stride(0), x.stride(1), x.stride(2))
    D.q_stride, D.k_stride, D.v_stride, D.o_stride = s3(q), s3(k), s3(v), s3(o)
    D.o, D.to, D.lse, D.key_lens = ptr(o), ptr(to), ptr(lse), ptr(key_lens)
    ws_bytes = lib.cosmos_attn_workspace_bytes(ctypes.byref(D))
    ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
    stream = torch.cuda.current_stream().cuda_stream
    ev = lambda: torch.cuda.Event(enable_timing=True)
    pack_ms, run_ms = [], []
    for i in range(warmup + steps):
        e0, e1, e2 = ev(), ev(), ev()
        e0.record()
        assert lib.cosmos_attn_pack_kv(ctypes.byref(D), ws.data_ptr(), ws_bytes, stream) == 0
        e1.record()
        # the one-call entry point (what the Python host uses) may cut a thin last round of workgroups along the keys;
        # pack + run never does.  So time that call and take the re-tiling, timed just before, out of it.
        assert lib.cosmos_attn_fwd_jvp(ctypes.byref(D), ws.data_ptr(), ws_bytes, stream) == 0
        e2.record()
        torch.cuda.synchronize()
        if i >= warmup:
            pack_ms.append(e0.elapsed_time(e1))
            run_ms.append(e1.elapsed_time(e2) - e0.elapsed_time(e1))
    run_avg = sum(run_ms) / len(run_ms)
    pack_avg = sum(pack_ms) / len(pack_ms)

    what = {"none": "attn fwd", "q": "attn fwd+JVP (tangent on q)", "full": "attn fwd+JVP"}[tangents]
    where = {"c2": "2B 480p (L=37440)", "c3": "2B 720p (L=84480)", "c4": "14B 720p (H=40, L=84480)",
             "c5": "2B text cross-attention (Lq=37440, Lkv<=512, key padding)"}[name]
    traffic, traffic_source = MEASURED_TRAFFIC_BYTES.get(name, _NO_TRAFFIC)
    # key padding: the FLOP that count are those of the valid keys and of the matmuls that are not identically zero
    # (the nominal figure -- 6 matmuls over the padded Lkv -- is kept beside it in `config`)
    flops_value = flops_alg if padded else flops
    alg_bytes = sum(x.numel() * x.element_size() for x in (q, k, v, tq, tk, tv, o, to, lse) if x is not None)
    roofline = {"bound": "mfma", "achieved": flops_value / (run_avg * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s"}
    if padded:
        # intensity = algorithmic FLOP / algorithmic bytes is below the ridge (peak FLOP/s / peak B/s): HBM-bound
        roofline = {"bound": "hbm", "achieved": alg_bytes / (run_avg * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "mfma_frac": flops_value / (run_avg * 1e-3) / 1e12 / PEAK_BF16_TFLOPS}
    roofline.update({"frac": roofline["achieved"] / roofline["peak"], "traffic": traffic, "traffic_source": traffic_source,
                     "algorithmic_bytes": alg_bytes,
                     "kernel": "attn_qstream_kernel" if name == "c5" else
                               ("attn_fwd_sym_kernel" if tangents == "none" and not padded else "attn_fwd_jvp_kernel") + " (+ attn_combine_kernel)",
                     "kernel_ms_avg": run_avg, "kernel_ms_min": min(run_ms),
                     "kernel_ms_median": sorted(run_ms)[len(run_ms) // 2], "pack_kv_kernel_ms_avg": pack_avg})
    result = {
        "metric": f"{what} TFLOP/s & % bf16 MFMA peak @ {where}; ms per call",
        "value": flops_value / sec / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": sec * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": desc_txt, "B": B, "H": H, "Lq": Lq, "Lkv": Lkv, "d": d,
                   "tangents": tangents, "flop_per_call": flops_value,
                   "pct_of_bf16_mfma_peak": 100.0 * flops_value / sec / 1e12 / PEAK_BF16_TFLOPS},
        "roofline": roofline,
    }
    if padded:
        result["config"]["mean_key_len"] = mean_len
        result["config"]["nominal_flop_per_call"] = flops
        result["config"]["nominal_tflops"] = flops / sec / 1e12
        result["config"]["step"] = "run_packed against a context image packed once (pack_kv outside the timed region)"
        result["ms_per_step_one_call"] = sec_one_call * 1e3
    # parity of the timed call's own output (the last timed step), all heads in play: sampled 128-row blocks against the
    # fp32 row-block oracle on the host -- outside the timed region
    del ws, o, to
    oracle = entry.load_oracle()
    result["parity_sampled"] = sampled_parity(oracle, (q, k, v, tq, tk, tv), out_timed, None if key_lens is None else key_lens.cpu().tolist(),
                                              n_blocks=8 if full else 4)
    if not full:
        return result
    if args.copy_calib:
        copy_calibration(dev)
    if args.gemm_ref:
        result["gemm_ref"] = gemm_reference(dev)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(oracle, H, Lkv, d, tangents)
    return result


if __name__ == "__main__":
    main()
