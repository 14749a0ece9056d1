"""Host-side plumbing shared by the three entry points: argument checks of the reference wrappers,
layout normalisation, parameter-block filling and the launch through the C ABI."""
from __future__ import annotations

import ctypes
from typing import Optional

import torch
import torch.nn.functional as F

from . import _capi

_TORCH_TO_ENUM = {torch.float16: _capi.INTFA_F16, torch.bfloat16: _capi.INTFA_BF16, torch.float32: _capi.INTFA_F32}
BLOCK = 128          # query block of the kernels
_VARIANT_ENUM = {"full": _capi.VARIANT_FULL_INT8, "half": _capi.VARIANT_HALF_INT8, "fp": _capi.VARIANT_FP16}


def block_n(variant: str, head_dim: int) -> int:
    """Key-block length the kernel of `variant` ("full", "half", "fp") uses at `head_dim` (the reference's BLOCK_N)."""
    rc = _capi.load().intfa_fwd_block_n(_VARIANT_ENUM[variant], max(int(head_dim), MIN_HEAD_DIM))
    if rc < 0:
        _capi.check(rc, "intfa_fwd_block_n")
    return rc
MIN_HEAD_DIM = 64    # smaller head dims are zero-padded up to this (QK^T and the kept output columns are unchanged)


def check_head_dims(q, k, v):
    """The reference's shape constraints (flash_atten_full_int8.py:189-193)."""
    hq, hk, hv = q.shape[-1], k.shape[-1], v.shape[-1]
    assert hq == hk and hk == hv
    assert hk in {16, 32, 64, 128, 256}
    return hk


def _rowmajor(t: torch.Tensor, elem_bytes: int) -> torch.Tensor:
    """Returns t if its head dim is contiguous and every other stride is 16-byte aligned, else a contiguous copy."""
    ok = t.stride(-1) == 1 and all((s * elem_bytes) % 16 == 0 for s in t.stride()[:-1]) and t.data_ptr() % 16 == 0
    return t if ok else t.contiguous()


def _pad_head_dim(t: torch.Tensor, d_to: int) -> torch.Tensor:
    d = t.shape[-1]
    return t if d == d_to else F.pad(t, (0, d_to - d))


def _can_fold(t: torch.Tensor, n: int) -> bool:
    """True if the rows of consecutive heads of t ([Z, H, N, ...]) lie at one constant stride."""
    return n == 1 or t.stride(1) == n * t.stride(2)


def _require_gpu(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("int_flashattention_amd kernels run on the GPU only; got a CPU tensor")


def launch_forward(variant: str, q, k, v, q_scale, k_scale, v_scale, causal: bool, sm_scale: float, out_dtype,
                   num_splits: int = 1, p_round: int = _capi.PROUND_REFERENCE, return_lse: bool = False,
                   v_scale_block: Optional[int] = None, seqlens_k: Optional[torch.Tensor] = None):
    lib = _capi.load()
    _require_gpu(q, k, v, q_scale, k_scale, v_scale)
    d = check_head_dims(q, k, v)
    Z, H, N, _ = q.shape
    H_kv = k.shape[1]
    N_k = k.shape[2]
    if k.shape[0] != Z or v.shape[0] != Z or v.shape[2] != N_k or v.shape[1] != H_kv:
        raise ValueError("q, k and v must share the batch size, and k and v their heads and length")
    if H % H_kv != 0:
        raise ValueError(f"the number of query heads ({H}) must be a multiple of the number of K/V heads ({H_kv})")
    dk = max(d, MIN_HEAD_DIM)
    qk_bytes = 1 if variant in ("full", "half") else 2
    v_bytes = 1 if variant == "full" else 2
    q_, k_, v_ = (_rowmajor(_pad_head_dim(t, dk), b) for t, b in ((q, qk_bytes), (k, qk_bytes), (v, v_bytes)))
    out = torch.empty((Z, H, N, dk), dtype=out_dtype, device=q.device)
    lse = torch.empty((Z, H, N), dtype=torch.float32, device=q.device) if return_lse else None

    p = _capi.FwdParams()
    p.q, p.k, p.v, p.out = q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), out.data_ptr()
    p.lse = lse.data_ptr() if lse is not None else None
    for name, t in (("q", q_), ("k", k_), ("v", v_), ("o", out)):
        setattr(p, f"{name}_stride_b", t.stride(0)); setattr(p, f"{name}_stride_h", t.stride(1)); setattr(p, f"{name}_stride_n", t.stride(2))
    keep = [q_, k_, v_]
    if variant in ("full", "half"):
        if q_scale.dtype != k_scale.dtype:
            k_scale = k_scale.to(q_scale.dtype)
        if q_scale.dtype not in _TORCH_TO_ENUM:
            raise TypeError(f"unsupported scale dtype {q_scale.dtype}")
        p.scale_dtype = _TORCH_TO_ENUM[q_scale.dtype]
        p.q_scale, p.k_scale = q_scale.data_ptr(), k_scale.data_ptr()
        p.qs_stride_b, p.qs_stride_h, p.qs_stride_n = q_scale.stride()
        p.ks_stride_b, p.ks_stride_h, p.ks_stride_n = k_scale.stride()
        keep += [q_scale, k_scale]
    if variant == "full":
        if v_scale.dim() == 4:
            vs = v_scale.float()                                     # blocked scales cross the ABI as fp32
            # one scale per block of keys and channel ([Z, H_kv, ceil(N_k / v_scale_block), d])
            vsb = block_n("full", d) if v_scale_block is None else int(v_scale_block)
            if vsb <= 0 or tuple(vs.shape) != (Z, H_kv, (N_k + vsb - 1) // vsb, d):
                raise ValueError(f"a blocked v_scale must be [Z, H_kv, ceil(N_k / {vsb}), d], got {tuple(vs.shape)}")
            vs = _pad_head_dim(vs, dk)
            if vs.stride(-1) != 1:
                vs = vs.contiguous()
            p.v_scale_block = vsb
            p.vs_stride_b, p.vs_stride_h, p.vs_stride_blk = vs.stride()[:3]
        else:
            if v_scale_block is not None:
                raise ValueError("v_scale_block needs a 4-D v_scale")
            vs = v_scale if v_scale.dtype == q_scale.dtype else v_scale.to(q_scale.dtype)
            p.vs_stride_b, p.vs_stride_h = vs.stride()
        p.v_scale = vs.data_ptr()
        keep.append(vs)
    p.batch, p.heads, p.seqlen, p.head_dim = Z, H, N, dk
    p.heads_kv = H_kv
    p.seqlen_k = N_k
    if seqlens_k is not None:
        # number of keys per batch entry (a cache filled to different lengths); int32 [Z] on the device
        _require_gpu(seqlens_k)
        if seqlens_k.dtype != torch.int32 or tuple(seqlens_k.shape) != (Z,):
            raise ValueError(f"seqlens_k must be an int32 tensor of shape ({Z},)")
        seqlens_k = seqlens_k.contiguous()
        p.seqlens_k = seqlens_k.data_ptr()
        keep.append(seqlens_k)
    # Few queries per head with grouped K/V heads (decoding): the g query heads of a group become g*N rows of ONE head,
    # so that a group streams its K/V once instead of g times.  Pure re-striding: same memory, same results per row.
    g = H // H_kv
    # (with the causal mask only where the kernel can be told the position of a row: the decode-shaped calls)
    decode_kernel = not (dk == 128 and p.v_scale_block == 64)     # (64-key scale rows under the 128-key block: general kernel)
    fold_rows = 2 * BLOCK if not causal else (64 if decode_kernel else 0)
    if g > 1 and g * N <= fold_rows and _can_fold(q_, N) and (variant == "fp" or _can_fold(q_scale, N)):
        if causal:
            p.causal_rows = N
        p.heads, p.heads_kv, p.seqlen = H_kv, H_kv, g * N
        p.q_stride_h, p.q_stride_n = g * q_.stride(1), (q_.stride(2) if N > 1 else q_.stride(1))
        p.o_stride_h = g * out.stride(1)
        if variant != "fp":
            p.qs_stride_h, p.qs_stride_n = g * q_scale.stride(1), (q_scale.stride(2) if N > 1 else q_scale.stride(1))
    p.io_dtype = _TORCH_TO_ENUM[out_dtype]
    p.causal = 1 if causal else 0
    p.sm_scale = float(sm_scale)
    p.p_round = p_round
    if num_splits == "auto":
        cus = torch.cuda.get_device_properties(q.device).multi_processor_count
        num_splits = lib.intfa_fwd_suggest_splits(ctypes.byref(p), _VARIANT_ENUM[variant], cus)
        if num_splits < 0:
            _capi.check(num_splits, "intfa_fwd_suggest_splits")
    p.num_splits = int(num_splits)
    ws = None
    if p.num_splits > 1:
        need = lib.intfa_fwd_workspace_bytes(ctypes.byref(p))
        ws = torch.empty((need,), dtype=torch.uint8, device=q.device)
        p.workspace, p.workspace_bytes = ws.data_ptr(), need
    stream = torch.cuda.current_stream(q.device).cuda_stream
    fn = {"full": lib.intfa_fwd_full_int8, "half": lib.intfa_fwd_half_int8, "fp": lib.intfa_fwd_fp16}[variant]
    with torch.cuda.device(q.device):
        rc = fn(ctypes.byref(p), ctypes.c_void_p(stream))
    _capi.check(rc, fn.__name__)
    for t in keep + ([ws] if ws is not None else []):
        t.record_stream(torch.cuda.current_stream(q.device))
    o = out if dk == d else out[..., :d].contiguous()
    return (o, lse) if return_lse else o


def debug_qk_int32(q8: torch.Tensor, k8: torch.Tensor) -> torch.Tensor:
    """int32 accumulators S = Q8 K8^T as produced by the kernels' MFMA tile code ([Z,H,N,N])."""
    lib = _capi.load()
    _require_gpu(q8, k8)
    Z, H, N, d = q8.shape
    dk = max(d, MIN_HEAD_DIM)
    q_, k_ = _rowmajor(_pad_head_dim(q8, dk), 1), _rowmajor(_pad_head_dim(k8, dk), 1)
    N_k = k8.shape[2]
    s = torch.empty((Z, H, N, N_k), dtype=torch.int32, device=q8.device)
    p = _capi.FwdParams()
    p.q, p.k = q_.data_ptr(), k_.data_ptr()
    p.q_stride_b, p.q_stride_h, p.q_stride_n = q_.stride()[:3]
    p.k_stride_b, p.k_stride_h, p.k_stride_n = k_.stride()[:3]
    p.batch, p.heads, p.seqlen, p.head_dim = Z, H, N, dk
    p.seqlen_k = N_k
    p.scale_dtype, p.io_dtype = _capi.INTFA_F32, _capi.INTFA_F16
    stream = torch.cuda.current_stream(q8.device).cuda_stream
    with torch.cuda.device(q8.device):
        rc = lib.intfa_debug_qk_int32(ctypes.byref(p), ctypes.c_void_p(s.data_ptr()), ctypes.c_void_p(stream))
    _capi.check(rc, "intfa_debug_qk_int32")
    return s
