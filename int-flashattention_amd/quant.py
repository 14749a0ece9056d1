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
