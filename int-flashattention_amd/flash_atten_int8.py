"""Drop-in for the reference module of the same name: ``attention_int8`` (flash_atten_int8.py:181-217)."""
import torch

from ._host import launch_forward


def attention_int8(q, k, v, q_scale, k_scale, causal, sm_scale, *, num_splits=1, return_lse=False, seqlens_k=None):
    """Half-int8 attention forward: int8 q, k with per-token scales, v in fp16 (or bf16); output in v's dtype
    (fp16 in the reference, flash_atten_int8.py:188-189)."""
    return launch_forward("half", q, k, v, q_scale, k_scale, None, causal, sm_scale, v.dtype,
                          num_splits=num_splits, return_lse=return_lse, seqlens_k=seqlens_k)
