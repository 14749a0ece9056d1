#!/usr/bin/env python3
"""Writes tests/golden/attention_small.npz: seeded inputs of one small problem and the outputs of the CPU oracle for the
three variants (causal and non-causal, the kernels' key-block lengths).  The reference holds no vectors for this path and
was not imported; these fixtures freeze the oracle's own answers so that a later change to the oracle (or to the
kernels) that moves them is noticed.  Run from the repository root:  python tests/golden/make_golden.py"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import intfa_oracle as O  # noqa: E402


def main():
    B, H, N, D = 1, 1, 160, 64                      # N is not a multiple of the 128-row query block on purpose
    # (the full-int8 kernel's key block at head_dim 64 is 64: the reference admits none longer than head_dim,
    # flash_atten_full_int8.py:88)
    q, k, v, _ = O.make_inputs(B, H, N, D, seed=2024)
    q8, qs = O.quant_pertoken(q)
    k8, ks = O.quant_pertoken(k)
    v8, vs = O.quant_pertensor(v)
    sm = D ** -0.5
    out = dict(q=q.numpy(), k=k.numpy(), v=v.numpy(), q8=q8.numpy(), k8=k8.numpy(), v8=v8.numpy(),
               qs=qs.numpy(), ks=ks.numpy(), vs=vs.numpy(), sm_scale=np.float32(sm),
               s_int32=O.qk_int32(q8, k8).numpy())
    for causal in (False, True):
        tag = "causal" if causal else "dense"
        out[f"full_ref_{tag}"] = O.attention_full_int8(q8, k8, v8, qs, ks, vs, causal, sm, block_n=64).numpy()
        out[f"full_rne_{tag}"] = O.attention_full_int8(q8, k8, v8, qs, ks, vs, causal, sm, block_n=64, p_requant=O.p_requant_rne).numpy()
        out[f"half_{tag}"] = O.attention_int8(q8, k8, v, qs, ks, causal, sm, block_n=64).numpy()
        out[f"fp_{tag}"] = O.attention_fp(q, k, v, causal, sm, block_n=64).numpy()
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "attention_small.npz"), **out)
    print("wrote attention_small.npz:", {k_: v_.shape for k_, v_ in out.items() if hasattr(v_, "shape")})


if __name__ == "__main__":
    main()
