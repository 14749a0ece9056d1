"""The quantisers of the reference's harness (benchmark.py:96-107) on HIP kernels: ``quant_pertoken`` and
``quant_pertensor`` with the reference's signatures (X -> (int8 X, scale))."""
import ctypes

import torch

from . import _capi

_DT = {torch.float16: _capi.INTFA_F16, torch.bfloat16: _capi.INTFA_BF16}


def _prepare(x):
    if not x.is_cuda:
        raise RuntimeError("int_flashattention_amd quantisers run on the GPU only; got a CPU tensor")
    if x.dtype not in _DT:
        raise TypeError(f"quantisers take fp16 or bf16 tensors, got {x.dtype}")
    if x.dim() != 4:
        raise ValueError("expected a [Z, H, N, d] tensor")
    ok = x.stride(-1) == 1 and all((s * 2) % 16 == 0 for s in x.stride()[:-1]) and x.data_ptr() % 16 == 0
    return x if ok else x.contiguous()


def quant_pertoken(x):
    """Per-row symmetric int8 (benchmark.py:96-100): scale = absmax / 127 in x's dtype, round-half-even."""
    lib = _capi.load()
    x_ = _prepare(x)
    Z, H, N, d = x_.shape
    q8 = torch.empty((Z, H, N, d), dtype=torch.int8, device=x.device)
    scale = torch.empty((Z, H, N), dtype=x.dtype, device=x.device)
    stream = torch.cuda.current_stream(x.device).cuda_stream
    with torch.cuda.device(x.device):
        rc = lib.intfa_quant_pertoken(x_.data_ptr(), x_.stride(0), x_.stride(1), x_.stride(2), q8.data_ptr(),
                                      scale.data_ptr(), Z, H, N, d, _DT[x.dtype], ctypes.c_void_p(stream))
    _capi.check(rc, "intfa_quant_pertoken")
    x_.record_stream(torch.cuda.current_stream(x.device))
    return q8, scale


def quant_pertensor(x):
    """One scale per (batch, head) slice (benchmark.py:102-107)."""
    lib = _capi.load()
    x_ = _prepare(x)
    Z, H, N, d = x_.shape
    q8 = torch.empty((Z, H, N, d), dtype=torch.int8, device=x.device)
    scale = torch.empty((Z, H), dtype=x.dtype, device=x.device)
    need = lib.intfa_quant_pertensor_workspace_bytes(Z, H)
    ws = torch.empty((need,), dtype=torch.uint8, device=x.device)
    stream = torch.cuda.current_stream(x.device).cuda_stream
    with torch.cuda.device(x.device):
        rc = lib.intfa_quant_pertensor(x_.data_ptr(), x_.stride(0), x_.stride(1), x_.stride(2), q8.data_ptr(),
                                       scale.data_ptr(), Z, H, N, d, _DT[x.dtype], ws.data_ptr(), need,
                                       ctypes.c_void_p(stream))
    _capi.check(rc, "intfa_quant_pertensor")
    for t in (x_, ws):
        t.record_stream(torch.cuda.current_stream(x.device))
    return q8, scale


def quant_perblock_channel(x, block):
    """One fp32 scale per (batch, head, block of ``block`` rows, channel) - the layout of the V scales that the
    reference's CUDA kernel reads (csrc/flash_fwd_kernel_full_qi8.h:156-160) - with the harness's formula
    (benchmark.py:102-107: absmax / 127, round-half-even) evaluated in fp32.  Returns (int8 [Z,H,N,d], fp32
    [Z,H,ceil(N/block),d]); pass both to ``attention_full_int8(..., v_scale_block=block)``."""
    lib = _capi.load()
    x_ = _prepare(x)
    Z, H, N, d = x_.shape
    block = int(block)
    if block <= 0:
        raise ValueError("block must be positive")
    q8 = torch.empty((Z, H, N, d), dtype=torch.int8, device=x.device)
    scale = torch.empty((Z, H, (N + block - 1) // block, d), dtype=torch.float32, device=x.device)
    stream = torch.cuda.current_stream(x.device).cuda_stream
    with torch.cuda.device(x.device):
        rc = lib.intfa_quant_perblock_channel(x_.data_ptr(), x_.stride(0), x_.stride(1), x_.stride(2), q8.data_ptr(),
                                              scale.data_ptr(), Z, H, N, d, block, _DT[x.dtype], ctypes.c_void_p(stream))
    _capi.check(rc, "intfa_quant_perblock_channel")
    x_.record_stream(torch.cuda.current_stream(x.device))
    return q8, scale


def kvcache_append(k_cache, k_scale_cache, k_new, seqlens_k, v_cache=None, v_scale=None, v_new=None):
    """Quantises new keys (and values) into an int8 K/V cache in place, at each batch entry's fill position: the
    quantised-cache counterpart of the knew/vnew copy of the reference's cache kernel (csrc/flash_fwd_kernel.h:690-790).

    k_cache, v_cache: int8 [Z, H_kv, N_cache, d]; k_scale_cache: [Z, H_kv, N_cache] and v_scale: [Z, H_kv] in k_new's
    dtype; k_new, v_new: fp16/bf16 [Z, H_kv, N_new, d]; seqlens_k: int32 [Z] on the device (rows already filled) or an
    int for all entries.  K rows are quantised per token like ``quant_pertoken`` (their scales land in
    ``k_scale_cache``); V rows with the cache's existing ``v_scale`` (saturating at +-127).  Rows past the end of the
    cache are dropped.  The lengths are not advanced here: pass ``seqlens_k + N_new`` to the next forward call."""
    lib = _capi.load()
    if not (k_cache.is_cuda and k_scale_cache.is_cuda and k_new.is_cuda):
        raise RuntimeError("int_flashattention_amd.kvcache_append runs on the GPU only; got a CPU tensor")
    if k_new.dtype not in _DT:
        raise TypeError(f"new keys must be fp16 or bf16, got {k_new.dtype}")
    if k_cache.dtype != torch.int8 or k_scale_cache.dtype != k_new.dtype:
        raise TypeError("k_cache must be int8 and k_scale_cache of k_new's dtype")
    Z, H, Nn, d = k_new.shape
    if k_cache.dim() != 4 or k_cache.shape[0] != Z or k_cache.shape[1] != H or k_cache.shape[3] != d:
        raise ValueError("k_cache must be [Z, H_kv, N_cache, d] with k_new's Z, H_kv and d")
    Nc = k_cache.shape[2]
    if tuple(k_scale_cache.shape) != (Z, H, Nc):
        raise ValueError("k_scale_cache must be [Z, H_kv, N_cache]")
    if k_cache.stride(-1) != 1:
        raise ValueError("k_cache rows must be contiguous (the append writes in place)")
    keep = []
    kn = _prepare(k_new); keep.append(kn)
    a = _capi.AppendParams()
    a.k_new = kn.data_ptr(); a.kn_stride_b, a.kn_stride_h, a.kn_stride_n = kn.stride(0), kn.stride(1), kn.stride(2)
    a.k_cache = k_cache.data_ptr(); a.kc_stride_b, a.kc_stride_h, a.kc_stride_n = k_cache.stride(0), k_cache.stride(1), k_cache.stride(2)
    a.k_scale_cache = k_scale_cache.data_ptr()
    a.ksc_stride_b, a.ksc_stride_h, a.ksc_stride_n = k_scale_cache.stride()
    if v_new is not None:
        if v_cache is None or v_scale is None:
            raise ValueError("v_new needs v_cache and v_scale")
        if v_new.dtype != k_new.dtype or v_scale.dtype != k_new.dtype or v_cache.dtype != torch.int8:
            raise TypeError("v_new and v_scale must have k_new's dtype, v_cache must be int8")
        if tuple(v_new.shape) != (Z, H, Nn, d) or tuple(v_cache.shape) != (Z, H, Nc, d) or tuple(v_scale.shape) != (Z, H):
            raise ValueError("v_new / v_cache / v_scale shapes do not match the keys'")
        if v_cache.stride(-1) != 1:
            raise ValueError("v_cache rows must be contiguous (the append writes in place)")
        vn = _prepare(v_new); keep.append(vn)
        a.v_new = vn.data_ptr(); a.vn_stride_b, a.vn_stride_h, a.vn_stride_n = vn.stride(0), vn.stride(1), vn.stride(2)
        a.v_cache = v_cache.data_ptr(); a.vc_stride_b, a.vc_stride_h, a.vc_stride_n = v_cache.stride(0), v_cache.stride(1), v_cache.stride(2)
        a.v_scale = v_scale.data_ptr(); a.vs_stride_b, a.vs_stride_h = v_scale.stride()
    if isinstance(seqlens_k, int):
        a.seqlens_k = None; a.seqlen_filled = seqlens_k
    else:
        if seqlens_k.dtype != torch.int32 or not seqlens_k.is_cuda or tuple(seqlens_k.shape) != (Z,) or not seqlens_k.is_contiguous():
            raise ValueError("seqlens_k must be a contiguous int32 [Z] tensor on the device (or an int)")
        a.seqlens_k = seqlens_k.data_ptr(); a.seqlen_filled = 0
    a.batch, a.heads_kv, a.seqlen_new, a.seqlen_cache, a.head_dim, a.dtype = Z, H, Nn, Nc, d, _DT[k_new.dtype]
    stream = torch.cuda.current_stream(k_new.device).cuda_stream
    with torch.cuda.device(k_new.device):
        rc = lib.intfa_kvcache_append_int8(ctypes.byref(a), ctypes.c_void_p(stream))
    _capi.check(rc, "intfa_kvcache_append_int8")
    for t in keep:
        t.record_stream(torch.cuda.current_stream(k_new.device))
