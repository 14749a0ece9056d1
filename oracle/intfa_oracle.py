"""CPU oracle for the INT8 FlashAttention forward path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain PyTorch on the CPU, the arithmetic that the reference's three
forward entry points perform.  It is the checker for the HIP kernels: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import it.  The product
package never does, and it fails loudly when its HIP library is missing.

What each function follows in the reference (paths relative to the reference checkout):

* ``quant_pertoken``           - benchmark.py:96-100
* ``quant_pertensor``          - benchmark.py:102-107
* ``mean_relative_error``      - benchmark.py:110-122 (``calc_num=4`` reproduces it; ``None`` = all elements)
* ``attention_exact``          - benchmark.py:152-154 (non-causal) and benchmark.py:224-230 (causal tril mask)
* ``qk_int32``                 - flash_atten_full_int8.py:36 (the int32 accumulator of ``tl.dot(q, k)``)
* ``attention_full_int8``      - flash_atten_full_int8.py:9-71 (tile loop), :148-182 (init + epilogue); the causal
                                 hand-off of the running max follows flash_atten_int8.py:66,157,166 because the
                                 full-int8 file drops it (flash_atten_full_int8.py:71,166,175 return only acc, l_i)
* ``attention_int8``           - flash_atten_int8.py:9-66, :140-176 (also returns M = m + log2(l), :172-175)
* ``attention_fp``             - flash_atten_fp.py:9-60, :115-150
* ``quant_perblock_channel``   - no quantiser for this layout exists in the reference; it applies the harness's formula
                                 (benchmark.py:102-107: absmax / 127, round-half-even) at the granularity of the V scale
                                 tensor its CUDA kernel reads (csrc/flash_fwd_kernel_full_qi8.h:156-160: one fp32 scale
                                 per key block and channel)
* ``attention_full_int8`` with a 4-D ``v_scale`` - the per-block, per-channel dequantisation of P V of that kernel
                                 (csrc/mask.h:313-340: acc_o += scale_col[col] * acc_o_int / 127)
* ``splitkv_ranges``           - csrc/flash_fwd_kernel.h:503-511 (key-block range of a split)
* ``splitkv_combine``          - csrc/flash_fwd_kernel.h:1212-1235 (log-sum-exp over splits), :1264-1283 (weighted sum)

Free parameters of the reference that are fixed here by argument: ``block_m``/``block_n`` (the reference
autotunes them, and its result depends on ``block_n`` because P is quantised against the running
maximum of the blocks seen so far) and the key-block order (ascending, as in the Triton loop).

How every function is pinned (tests/test_oracle.py):

* quantisers: closed form (absmax/127, round-half-even), invariants (every row reaches +-127), brute force.
* ``qk_int32``: exact integer matmul compared with a pure-Python triple loop and with numpy int64.
* P requantisation ``p_requant_reference``: exhaustive over all fp16 values in [0, 1] against a scalar
  restatement using ``numpy.float16`` arithmetic.
* online softmax: ``block_n = N`` must reproduce ``torch.softmax``; any ``block_n`` gives the same (m, l) up to
  fp32 rounding; with every scale equal to one the path is plain integer attention; with V constant the output
  is that constant times sum(P8)/(127 l).
* causal: equality with a dense tril-masked evaluation; first row attends to key 0 only.
* split-KV: any split count agrees with one split to fp32 rounding.
* separate query and key lengths: rows are independent, so a slice of the query rows against the full keys must
  reproduce the same rows of the square evaluation bit for bit; causal with the mask aligned to the bottom right corner:
  the last Nq rows of the square causal problem, bit for bit; with fewer keys than queries the first rows see nothing
  and give zeros.
* blocked V scales: a 4-D scale tensor filled with one value per (batch, head) reproduces the scalar form bit for
  bit; the result equals the scalar form applied to V pre-multiplied by the block/channel factors when these are
  powers of two; ``quant_perblock_channel`` against a pure-Python loop, and every (block, channel) reaches +-127.
* ``kvcache_append``: a cache filled by two appends equals the quantisers applied to the concatenation (K: rows are
  independent, bit for bit incl. scales; V: with the concatenation's per-tensor scale, bit for bit); values beyond the
  cache's V scale saturate at +-127; rows outside the appended range stay untouched; rows past the end are dropped.

The reference holds no golden vectors for this path (its only test asserts the fp16 forward with
atol=1e-2, benchmark.py:242), so none are used.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

LOG2E = 1.44269504  # the literal used at flash_atten_full_int8.py:157


# --------------------------------------------------------------------------------------------------
# quantisers and error measures (benchmark.py)
# --------------------------------------------------------------------------------------------------
def quant_pertoken(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """benchmark.py:96-100: per-row symmetric int8, scale = absmax/127 in the input dtype."""
    x_max, _ = torch.abs(x).max(dim=-1)
    x_scale = x_max / 127
    ret = torch.round(x / x_scale[:, :, :, None]).to(torch.int8)
    return ret, x_scale


def quant_pertensor(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """benchmark.py:102-107: one scale per (batch, head) slice."""
    x_max, _ = torch.abs(x).max(dim=-1)
    x_max, _ = torch.max(x_max, dim=-1)
    x_scale = x_max / 127
    ret = torch.round(x / x_scale[:, :, None, None]).to(torch.int8)
    return ret, x_scale


def kvcache_append(k_cache, k_scale_cache, k_new, seqlens_k, v_cache=None, v_scale=None, v_new=None) -> None:
    """Appends new keys (and values) to an int8 K/V cache in place: for batch entry b the rows go to positions
    len_b .. len_b + N_new - 1, len_b = seqlens_k[b] clamped to the cache (the copy of knew/vnew that the reference's
    cache kernel makes, csrc/flash_fwd_kernel.h:690-790, for a quantised cache); rows past the end of the cache are
    dropped.  K rows are quantised per token (``quant_pertoken``: the rows are independent, so this equals quantising
    the concatenation), their scales go to ``k_scale_cache``; V rows with the cache's existing per-(batch, head) scale,
    q = round-half-even(v / scale) in v's dtype saturated to [-127, 127] (0 / 0 gives 0)."""
    Z, _, n_new, _ = k_new.shape
    n_cache = k_cache.shape[2]
    k8, ks = quant_pertoken(k_new)
    for b in range(Z):
        n0 = min(max(int(seqlens_k[b]), 0), n_cache)
        n = min(n_new, n_cache - n0)
        k_cache[b, :, n0:n0 + n] = k8[b, :, :n]
        k_scale_cache[b, :, n0:n0 + n] = ks[b, :, :n]
        if v_new is not None:
            q = torch.round(v_new[b, :, :n] / v_scale[b][:, None, None])
            q = torch.where(torch.isnan(q), torch.zeros_like(q), q.clamp(-127, 127))
            v_cache[b, :, n0:n0 + n] = q.to(torch.int8)


def quant_perblock_channel(x: torch.Tensor, block: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """One fp32 scale per (batch, head, block of ``block`` rows, channel): scale = absmax / 127 over the block's rows,
    int8 = round-half-even(x / scale), both in fp32.  Returns (int8 [B,H,N,d], scale [B,H,ceil(N/block),d]).  A channel
    that is all zero inside a block gets scale 0 and int8 0."""
    B, H, N, D = x.shape
    nblk = (N + block - 1) // block
    xf = x.float()
    pad = nblk * block - N
    if pad:
        xf = torch.cat([xf, torch.zeros((B, H, pad, D))], dim=2)
    xb = xf.view(B, H, nblk, block, D)
    scale = xb.abs().amax(dim=3) / 127                                       # [B,H,nblk,D] fp32
    safe = torch.where(scale > 0, scale, torch.ones_like(scale))
    q = torch.round(xb / safe[:, :, :, None, :])
    q = torch.where(scale[:, :, :, None, :] > 0, q, torch.zeros_like(q))
    return q.view(B, H, nblk * block, D)[:, :, :N].to(torch.int8).contiguous(), scale


def mean_relative_error(a: torch.Tensor, b: torch.Tensor, calc_num: Optional[int] = None) -> float:
    """benchmark.py:110-122: mean(|b - a| / (|b| + 1e-5)); the reference looks at the last 4 elements only."""
    assert a.shape == b.shape
    m1 = b.reshape(-1).float()
    m2 = a.reshape(-1).float()
    if calc_num is not None:
        m1, m2 = m1[-calc_num:], m2[-calc_num:]
    return (torch.abs(m1 - m2) / (torch.abs(m1) + 1e-5)).mean().item()


def attention_exact(q, k, v, causal: bool, sm_scale: float) -> torch.Tensor:
    """benchmark.py:152-154 / :224-230: softmax(QK^T * sm_scale) V with an fp32 softmax.

    Computed in fp32 throughout on the CPU (the reference does the two matmuls in fp16 on the GPU);
    P is rounded to the input dtype before the second matmul as the reference does.
    """
    qf, kf, vf = q.float(), k.float(), v.float()
    p = torch.matmul(qf, kf.transpose(2, 3)) * sm_scale
    if causal:
        n, nk = q.shape[2], k.shape[2]           # equal in the reference; otherwise the mask is aligned bottom right
        mask = (torch.arange(n)[:, None] + (nk - n)) >= torch.arange(nk)[None, :]
        p = p.masked_fill(~mask, float("-inf"))
    p = torch.softmax(p, dim=-1).to(q.dtype if q.dtype.is_floating_point else torch.float16).float()
    return torch.matmul(p, vf).to(q.dtype if q.dtype.is_floating_point else torch.float16)


# --------------------------------------------------------------------------------------------------
# integer pieces
# --------------------------------------------------------------------------------------------------
def _int_matmul(a8: torch.Tensor, b8: torch.Tensor) -> torch.Tensor:
    """Exact integer matmul a8 @ b8 returned as fp32 holding integers.

    fp32 GEMM is exact here: every partial sum is an integer below 2**24 (|a|,|b| <= 128, inner
    dimension <= 1024), so no rounding occurs in any summation order.
    """
    assert a8.shape[-1] <= 1024
    return torch.matmul(a8.float(), b8.float())


def qk_int32(q8: torch.Tensor, k8: torch.Tensor) -> torch.Tensor:
    """flash_atten_full_int8.py:36: S = Q8 K8^T accumulated in int32, shape [B,H,N,N]."""
    return _int_matmul(q8, k8.transpose(2, 3)).to(torch.int32)


def p_requant_reference(p: torch.Tensor) -> torch.Tensor:
    """flash_atten_full_int8.py:49-51: p.to(fp16); p * 127; (p + 0.5).to(int8) - all in fp16, truncating cast.

    Returns fp32 holding the integers 0..127.
    """
    p16 = p.to(torch.float16)
    p16 = p16 * 127          # fp16 product, rounded to fp16
    p16 = p16 + 0.5          # fp16 sum, rounded to fp16
    return torch.trunc(p16.float())


def p_requant_rne(p: torch.Tensor) -> torch.Tensor:
    """Round-to-nearest-even of 127 p in fp32: what one hardware float->u8 convert of 127 p yields.

    Not the reference's formula; kept so tests can measure how far the two roundings are apart.
    """
    return torch.clamp(torch.round(p * 127.0), 0, 255)


# --------------------------------------------------------------------------------------------------
# the blocked forward (all three variants share the loop skeleton)
# --------------------------------------------------------------------------------------------------
def _blocked_forward(variant: str, q, k, v, q_scale, k_scale, v_scale, causal: bool, sm_scale: float,
                     block_m: int, block_n: int, key_lo: int = 0, key_hi: Optional[int] = None,
                     p_requant=p_requant_reference, pv_dtype=torch.float16,
                     row_lo: int = 0, row_hi: Optional[int] = None, v_scale_block: Optional[int] = None):
    """Runs the reference's tile loop over key blocks [key_lo, key_hi) for every query row at once.

    Rows are grouped in tiles of ``block_m`` as the reference's programs are; for a causal run a tile sees
    the key blocks below its first row without a mask (stage 1) and the blocks of its own row range with the
    mask (stage 2), flash_atten_full_int8.py:18-25.  Returns fp32 (acc, l, m) with acc un-normalised.
    Only rows [row_lo, row_hi) are evaluated (the others keep m = -inf, l = 1, acc = 0).
    A 4-D ``v_scale`` [B,H,ceil(N/v_scale_block),d] selects the per-block, per-channel dequantisation of P V
    (csrc/mask.h:313-340); ``v_scale_block`` must be a multiple of ``block_n`` or divide it.  When it divides it (64-key
    scale rows, the reference kernel's kBlockN, under a 128-key softmax block) the int32 P V is formed per scale row and
    each partial sum is multiplied by its own row before it joins the accumulator, in ascending key order - what the
    reference's kernel does block by block (csrc/mask.h:335-336) with the block maximum of the larger block.
    """
    B, H, N, D = q.shape
    Nk = k.shape[2]                # differs from N for cross attention / a chunk of new tokens against a cache
    # causal: row i sees keys 0 .. i + off.  off = 0 is the reference's Python API (one N_CTX, flash_atten_full_int8.py:213);
    # with more keys than queries the mask is aligned to the bottom right corner as in its CUDA tree (csrc/mask.h:53,172:
    # col_idx_limit_right = row_idx + 1 + max_seqlen_k - max_seqlen_q)
    off = Nk - N
    key_hi = Nk if key_hi is None else key_hi
    row_hi = N if row_hi is None else row_hi
    # N need not be a multiple of the blocks: the last key block and the last row tile are simply shorter, which is
    # what masking the missing keys with -inf amounts to (csrc/mask.h:261-263 for the reference's CUDA tree; its Triton
    # kernels have no bounds handling at all)
    assert block_m % block_n == 0
    assert key_lo % block_n == 0 and (key_hi % block_n == 0 or key_hi == Nk)
    qk_scale = float(torch.tensor(sm_scale, dtype=torch.float32) * torch.tensor(LOG2E, dtype=torch.float32))
    m = torch.full((B, H, N), float("-inf"), dtype=torch.float32)
    l = torch.ones((B, H, N), dtype=torch.float32)          # flash_atten_full_int8.py:153
    acc = torch.zeros((B, H, N, D), dtype=torch.float32)
    int_qk = variant in ("full", "half")
    if int_qk:
        qs = q_scale.float()
        ks = k_scale.float()
    vs_blocked = variant == "full" and v_scale.dim() == 4
    if vs_blocked:
        v_scale_block = block_n if v_scale_block is None else v_scale_block
        assert (v_scale_block % block_n == 0 or block_n % v_scale_block == 0)
        assert v_scale.shape[2] == (Nk + v_scale_block - 1) // v_scale_block
    elif variant == "full":
        vs = v_scale.float()[:, :, None, None]
    rows = torch.arange(N)

    for start_n in range(key_lo, key_hi, block_n):
        kj = k[:, :, start_n:start_n + block_n]
        vj = v[:, :, start_n:start_n + block_n]
        if causal and off == 0:
            tile = start_n // block_m
            segments = [(tile * block_m, min((tile + 1) * block_m, N), True), ((tile + 1) * block_m, N, False)]
        elif causal:
            # rows that see a part of this block (masked evaluation) and rows that see all of it; rows above see nothing.
            # (For rows that see the whole block the two evaluations give identical numbers, so where the boundary
            # between the segments lies does not matter.)
            end_n = min(start_n + block_n, key_hi)
            lo, hi = min(max(start_n - off, 0), N), min(max(end_n - off, 0), N)
            segments = [(lo, hi, True), (hi, N, False)]
        else:
            segments = [(0, N, False)]
        for r0, r1, masked in segments:
            r0, r1 = max(r0, row_lo), min(r1, row_hi)
            if r0 >= r1:
                continue
            qi = q[:, :, r0:r1]
            if int_qk:
                qk = _int_matmul(qi, kj.transpose(2, 3))                     # int32 accumulator, :36
                qk = qk * qs[:, :, r0:r1, None]                              # :37
                qk = qk * ks[:, :, None, start_n:start_n + block_n]          # :38
            else:
                qk = torch.matmul(qi.float(), kj.float().transpose(2, 3))    # flash_atten_fp.py:33
            m_i = m[:, :, r0:r1]
            if masked:                                                       # :39-43
                keep = (rows[r0:r1, None] + off) >= (start_n + torch.arange(kj.shape[2]))[None, :]
                qk = qk * qk_scale + torch.where(keep, 0.0, -1.0e6)
                m_ij = torch.maximum(m_i, qk.max(dim=-1).values)
                qk = qk - m_ij[..., None]
            else:                                                            # :44-46
                m_ij = torch.maximum(m_i, qk.max(dim=-1).values * qk_scale)
                qk = qk * qk_scale - m_ij[..., None]
            p = torch.exp2(qk)                                               # :47
            l_ij = p.sum(dim=-1)                                             # :48
            alpha = torch.exp2(m_i - m_ij)                                   # :53
            l[:, :, r0:r1] = l[:, :, r0:r1] * alpha + l_ij                   # :54
            a = acc[:, :, r0:r1] * alpha[..., None]                          # :56
            if variant == "full":
                p8 = p_requant(p)                                            # :49-51
                if vs_blocked and v_scale_block < block_n:                   # several scale rows inside this key block
                    for c0 in range(0, kj.shape[2], v_scale_block):
                        tmp = _int_matmul(p8[..., c0:c0 + v_scale_block], vj[:, :, c0:c0 + v_scale_block])
                        vs = v_scale.float()[:, :, (start_n + c0) // v_scale_block][:, :, None, :]
                        a = a + tmp * vs / 127                               # csrc/mask.h:335-336, one scale row at a time
                else:
                    tmp = _int_matmul(p8, vj)                                # :59 int32 accumulator
                    if vs_blocked:                                           # csrc/mask.h:335
                        vs = v_scale.float()[:, :, start_n // v_scale_block][:, :, None, :]
                    tmp = tmp * vs / 127                                     # :61
                    a = a + tmp                                              # :62
            else:
                pl = p.to(pv_dtype).float()                                  # flash_atten_int8.py:58
                a = a + torch.matmul(pl, vj.float())                         # :59 fp32 accumulate
            acc[:, :, r0:r1] = a
            m[:, :, r0:r1] = m_ij                                            # :67
    return acc, l, m


def attention_full_int8(q, k, v, q_scale, k_scale, v_scale, causal: bool, sm_scale: float, *,
                        block_m: int = 128, block_n: int = 128, out_dtype=torch.float16,
                        p_requant=p_requant_reference, return_lse: bool = False,
                        v_scale_block: Optional[int] = None):
    """Full-int8 forward, flash_atten_full_int8.py (see module docstring for line map).  ``v_scale`` is [B,H] (the
    reference's Python API) or [B,H,ceil(N/v_scale_block),d] (the layout of its CUDA kernel)."""
    acc, l, m = _blocked_forward("full", q, k, v, q_scale, k_scale, v_scale, causal, sm_scale,
                                 block_m, block_n, p_requant=p_requant, v_scale_block=v_scale_block)
    o = (acc / l[..., None]).to(out_dtype)                                   # :181-182
    if return_lse:
        return o, m + torch.log2(l)
    return o


def attention_int8(q, k, v, q_scale, k_scale, causal: bool, sm_scale: float, *,
                   block_m: int = 128, block_n: int = 128, out_dtype=torch.float16, return_lse: bool = False):
    """Half-int8 forward, flash_atten_int8.py: int8 QK^T, P cast to V's dtype, fp32-accumulated PV."""
    acc, l, m = _blocked_forward("half", q, k, v, q_scale, k_scale, None, causal, sm_scale,
                                 block_m, block_n, pv_dtype=v.dtype)
    o = (acc / l[..., None]).to(out_dtype)
    if return_lse:
        return o, m + torch.log2(l)                                          # :172-175
    return o


def attention_fp(q, k, v, causal: bool, sm_scale: float, *, block_m: int = 128, block_n: int = 128,
                 return_lse: bool = False):
    """fp16/bf16 forward, flash_atten_fp.py; output has q's dtype (:162)."""
    acc, l, m = _blocked_forward("fp", q, k, v, None, None, None, causal, sm_scale,
                                 block_m, block_n, pv_dtype=q.dtype)
    o = (acc / l[..., None]).to(q.dtype)
    if return_lse:
        return o, m + torch.log2(l)
    return o


# --------------------------------------------------------------------------------------------------
# split-KV (the reference has it for fp16 only; csrc/kernel_traits.h:199 leaves the int8 version open)
# --------------------------------------------------------------------------------------------------
def splitkv_ranges(n_keys: int, block_n: int, num_splits: int):
    """csrc/flash_fwd_kernel.h:503-511: key-block range [min, max) of each split."""
    n_blocks = (n_keys + block_n - 1) // block_n
    per = (n_blocks + num_splits - 1) // num_splits
    return [(s * per, min(n_blocks, (s + 1) * per)) for s in range(num_splits)]


def splitkv_combine(o_parts: torch.Tensor, lse_parts: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """csrc/flash_fwd_kernel.h:1212-1235, :1264-1283 in base 2 (the kernels keep log2-domain statistics).

    o_parts [S,B,H,N,D] fp32 are partial outputs already divided by their own l; lse_parts [S,B,H,N]
    are m + log2(l), -inf for a split that saw no key.
    """
    lse_max = lse_parts.max(dim=0).values
    empty = torch.isinf(lse_max) & (lse_max < 0)            # no split saw a key for this row
    lse_max = torch.where(empty, torch.zeros_like(lse_max), lse_max)
    lse_sum = torch.exp2(lse_parts - lse_max).sum(dim=0)
    # the weights of an empty row are zero (the reference gets there by setting the row's lse to +inf, :1226); the lse
    # REPORTED for such a row is -inf, as for a single pass over no key (the neutral element of a merge by lse)
    lse_w = torch.where(empty, torch.full_like(lse_sum, float("inf")), torch.log2(lse_sum) + lse_max)
    w = torch.exp2(lse_parts - lse_w)
    lse = torch.where(empty, torch.full_like(lse_sum, float("-inf")), lse_w)
    return (w[..., None] * o_parts).sum(dim=0), lse


def splitkv_ranges_causal(n_keys: int, block_m: int, block_n: int, num_splits: int):
    """Causal split-KV as the kernels do it: per row tile of block_m rows, the key blocks VISIBLE to the tile are dealt
    evenly to the splits.  Returns [(row_lo, row_hi, [(block_min, block_max) per split])] per tile."""
    n_blocks = (n_keys + block_n - 1) // block_n
    out = []
    for r0 in range(0, n_keys, block_m):
        vis = min((r0 + block_m + block_n - 1) // block_n, n_blocks)
        per = (vis + num_splits - 1) // num_splits
        out.append((r0, min(r0 + block_m, n_keys), [(s * per, min(vis, (s + 1) * per)) for s in range(num_splits)]))
    return out


def attention_full_int8_splitkv(q, k, v, q_scale, k_scale, v_scale, causal: bool, sm_scale: float, num_splits: int, *,
                                block_m: int = 128, block_n: int = 128, out_dtype=torch.float16,
                                v_scale_block: Optional[int] = None, p_requant=p_requant_reference):
    """Full-int8 forward evaluated as ``num_splits`` independent key ranges merged by ``splitkv_combine``: the ranges of
    ``splitkv_ranges`` for a non-causal pass, those of ``splitkv_ranges_causal`` (per row tile) for a causal one."""
    B, H, N, D = q.shape
    assert not causal or k.shape[2] == N      # the causal partition below is the one of equal lengths
    o_parts = torch.zeros((num_splits, B, H, N, D))
    lse_parts = torch.full((num_splits, B, H, N), float("-inf"))
    if causal:
        jobs = [(s, r0, r1, b0, b1) for r0, r1, ranges in splitkv_ranges_causal(N, block_m, block_n, num_splits)
                for s, (b0, b1) in enumerate(ranges)]
    else:
        jobs = [(s, 0, N, b0, b1) for s, (b0, b1) in enumerate(splitkv_ranges(k.shape[2], block_n, num_splits))]
    for s, r0, r1, b0, b1 in jobs:
        if b0 >= b1:
            continue
        acc, l, m = _blocked_forward("full", q, k, v, q_scale, k_scale, v_scale, causal, sm_scale,
                                     block_m, block_n, key_lo=b0 * block_n, key_hi=min(b1 * block_n, k.shape[2]),
                                     row_lo=r0, row_hi=r1, v_scale_block=v_scale_block, p_requant=p_requant)
        seen = ~torch.isinf(m[:, :, r0:r1])          # rows above the split's range saw no key
        a, ll, mm = acc[:, :, r0:r1], l[:, :, r0:r1], m[:, :, r0:r1]
        o_parts[s, :, :, r0:r1] = torch.where(seen[..., None], a / ll[..., None], torch.zeros_like(a))
        lse_parts[s, :, :, r0:r1] = torch.where(seen, mm + torch.log2(ll), torch.full_like(mm, float("-inf")))
    o, _ = splitkv_combine(o_parts, lse_parts)
    return o.to(out_dtype)


# --------------------------------------------------------------------------------------------------
# synthetic inputs of the benchmark configurations
# --------------------------------------------------------------------------------------------------
def make_inputs(B: int, H: int, N: int, D: int, *, seed: int = 20, dtype=torch.float16, std: float = 1.0,
                k_outlier_frac: float = 0.0, k_outlier_gain: float = 20.0):
    """Seeded N(0, std) Q, K, V in ``dtype``; optionally a fraction of K's channels is multiplied by a gain."""
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn((B, H, N, D), generator=g) * std).to(dtype)
    k = torch.randn((B, H, N, D), generator=g) * std
    v = (torch.randn((B, H, N, D), generator=g) * std).to(dtype)
    cols = []
    if k_outlier_frac > 0:
        n_out = max(1, int(round(D * k_outlier_frac)))
        cols = torch.randperm(D, generator=g)[:n_out].tolist()
        k[..., cols] *= k_outlier_gain
    return q, k.to(dtype), v, cols
