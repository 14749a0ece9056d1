"""Drop-in for the reference module of the same name: ``attention_full_int8`` (flash_atten_full_int8.py:186-223)."""
import torch

from . import _capi
from ._host import launch_forward


def attention_full_int8(q, k, v, q_scale, k_scale, v_scale, causal, sm_scale, *, out_dtype=torch.float16,
                        num_splits=1, p_round="reference", return_lse=False, v_scale_block=None, seqlens_k=None):
    """Full-int8 attention forward.

    q, k, v: int8 [Z, H, N, d]; q_scale, k_scale: [Z, H, N] per-token scales; v_scale: [Z, H];
    returns a new contiguous [Z, H, N, d] tensor, fp16 as in the reference (flash_atten_full_int8.py:194-195)
    unless ``out_dtype=torch.bfloat16`` is asked for.  Causal runs use the correct running-max hand-off between
    the off-diagonal and diagonal stages (as flash_atten_int8.py:157-166 does), not the reference's
    full-int8 behaviour, which restarts from -inf (flash_atten_full_int8.py:166,175).

    ``v_scale`` may also be 4-D, [Z, H, ceil(N / v_scale_block), d]: one scale per block of ``v_scale_block`` keys and
    channel, the V scales of the reference's CUDA kernel (csrc/flash_fwd_kernel_full_qi8.h:156-160), as produced by
    ``quant_perblock_channel``.  ``v_scale_block`` defaults to the kernel's key-block length (``block_n("full", d)``)
    and must be a multiple of it, or 64 at d <= 128 (the reference kernel's own block, kBlockN = 64,
    csrc/flash_fwd_launch_template.h:514-519).

    k and v may have another length than q (and fewer heads: grouped-query attention).  With ``causal`` query row i then
    sees keys 0 .. i + Nk - Nq (mask aligned to the bottom right corner: new tokens against a cache).
    ``seqlens_k`` (int32 [Z] on the device): number of keys of each batch entry when k and v are a cache filled to
    different lengths; rows past an entry's length are not read.

    ``p_round``: "reference" (the default) reproduces the fp16 sequence of flash_atten_full_int8.py:49-51 when P is
    requantised; "rne" is an opt-in that folds 127 into the exponent and rounds to nearest-even in fp32.
    """
    pr = {"rne": _capi.PROUND_RNE, "reference": _capi.PROUND_REFERENCE}[p_round]
    return launch_forward("full", q, k, v, q_scale, k_scale, v_scale, causal, sm_scale, out_dtype,
                          num_splits=num_splits, p_round=pr, return_lse=return_lse, v_scale_block=v_scale_block,
                          seqlens_k=seqlens_k)
