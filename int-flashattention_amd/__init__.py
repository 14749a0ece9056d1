"""MI355X-native INT8 FlashAttention forward behind the reference's Python entry points.

    attention(q, k, v, causal, sm_scale)
    attention_int8(q, k, v, q_scale, k_scale, causal, sm_scale)
    attention_full_int8(q, k, v, q_scale, k_scale, v_scale, causal, sm_scale)

All three launch hand-written HIP kernels (gfx950) through the C ABI of ``libintfa.so``; nothing here
computes attention in PyTorch.
"""
from .flash_atten_fp import attention
from .flash_atten_int8 import attention_int8
from .flash_atten_full_int8 import attention_full_int8
from ._host import debug_qk_int32, block_n
from .quant import quant_pertoken, quant_pertensor, quant_perblock_channel, kvcache_append

__all__ = ["attention", "attention_int8", "attention_full_int8", "debug_qk_int32", "block_n", "quant_pertoken", "quant_pertensor",
           "quant_perblock_channel", "kvcache_append"]
