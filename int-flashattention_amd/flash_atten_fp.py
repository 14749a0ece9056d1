"""Drop-in for the reference module of the same name: ``attention`` (flash_atten_fp.py:155-189)."""
from ._host import launch_forward


def attention(q, k, v, causal, sm_scale, *, num_splits=1, return_lse=False, seqlens_k=None):
    """fp16 (or bf16) attention forward; the output has q's dtype (flash_atten_fp.py:162)."""
    return launch_forward("fp", q, k, v, None, None, None, causal, sm_scale, q.dtype,
                          num_splits=num_splits, return_lse=return_lse, seqlens_k=seqlens_k)
