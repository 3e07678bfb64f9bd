"""GPU parity: the HIP forward + JVP through the C ABI against the CPU oracle on identical seeded inputs.

Tolerances (bf16 / fp16 inputs, fp32 oracle = torch math SDPA under torch.func.jvp):
max-abs <= 2e-2 and relative-L2 <= 5e-3 for O and dO; LSE max-abs <= 2e-3.
"""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ABS, REL_L2, LSE_ABS = 2e-2, 5e-3, 2e-3


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


def test_smallest(pkg, oracle, gpu):
    run_case(pkg, oracle, gpu, (1, 1, 64, 128))


def test_one_tile_ragged(pkg, oracle, gpu):
    run_case(pkg, oracle, gpu, (1, 2, 50, 128), (1, 2, 37, 128))


@pytest.mark.parametrize("L", [128, 192, 999, 1024])
def test_self_attention_d128(pkg, oracle, gpu, L):
    run_case(pkg, oracle, gpu, (1, 2, L, 128), seed=L)


def test_against_torch_sdpa_jvp(pkg, oracle, gpu):
    """The quoted oracle itself (torch math SDPA under torch.func.jvp, fp32) on a mid-size case."""
    q, k, v, tq, tk, tv = oracle.make_inputs((2, 3, 300, 128), seed=5)
    o, to = pkg.attention_jvp(*(x.to(gpu) for x in (q, k, v, tq, tk, tv)))
    o_ref, to_ref = oracle.sdpa_jvp_torch(q, k, v, tq, tk, tv)
    check(oracle, "o", o, o_ref)
    check(oracle, "to", to, to_ref)
