"""Writes the golden fixtures ``tests/golden/attn_jvp_golden.npz``.

The vectors come from the quoted oracle -- torch math ``scaled_dot_product_attention`` under
``torch.func.jvp`` in fp32 on CPU (``oracle/attention_oracle.py: sdpa_jvp_torch``) -- run in the build container
with torch 2.10.0.  No reference code is imported or executed; the reference holds no stored vectors for this
path (its JVP tests are commented-out procedures).  Inputs are regenerated from seeds by the tests, so only
the expected outputs (O, dO, fp32) and the LSE are stored.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import __graft_entry__ as entry  # noqa: E402

# name: (shape_q, shape_kv, dv, causal, sm_scale, key_lens, seed, dtype, primal_std, tangent_std, rms)
CASES = {
    "self_d128": ((1, 2, 96, 128), None, None, False, None, None, 11, "bf16", 1.0, 0.1, False),
    "self_d64_causal": ((1, 2, 130, 64), None, None, True, 0.5, None, 12, "bf16", 0.5, 0.5, False),
    "cross_ragged_dv32": ((1, 2, 70, 128), (1, 2, 15, 128), 32, False, 0.5, None, 13, "bf16", 0.5, 0.5, False),
    "cross_keypad": ((2, 2, 64, 128), (2, 2, 80, 128), None, False, None, [37, 80], 14, "bf16", 1.0, 0.1, False),
    "self_fp16_rms": ((1, 2, 70, 128), None, None, False, None, None, 15, "fp16", 1.0, 0.1, True),
    "fp32_plumbing_small": ((1, 1, 128, 128), None, None, False, None, None, 16, "fp32", 0.5, 0.5, False),
}
DTYPES = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def case_inputs(oracle, name):
    shape_q, shape_kv, dv, causal, sm_scale, key_lens, seed, dt, pstd, tstd, rms = CASES[name]
    tensors = oracle.make_inputs(shape_q, shape_kv, seed=seed, primal_std=pstd, tangent_std=tstd, rms_norm_qk=rms,
                                 dtype=DTYPES[dt], dv=dv)
    return tensors, dict(causal=causal, sm_scale=sm_scale, key_lens=key_lens)


def main():
    oracle = entry.load_oracle()
    out = {}
    for name in CASES:
        (q, k, v, tq, tk, tv), kw = case_inputs(oracle, name)
        if kw["causal"]:
            o, to = oracle.sdpa_jvp_torch(q, k, v, tq, tk, tv, sm_scale=kw["sm_scale"], causal=True)
        else:
            o, to = oracle.sdpa_jvp_torch(q, k, v, tq, tk, tv, sm_scale=kw["sm_scale"], key_lens=kw["key_lens"])
        _, _, lse = oracle.closed_form(q, k, v, tq, tk, tv, **kw)
        out[name + "/o"] = o.numpy().astype(np.float32)
        out[name + "/to"] = to.numpy().astype(np.float32)
        out[name + "/lse"] = lse.astype(np.float32)
    path = os.path.join(HERE, "attn_jvp_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
