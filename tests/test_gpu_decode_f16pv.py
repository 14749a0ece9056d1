"""GPU parity of the decode-shaped half-int8 and fp16/bf16 forward (few query rows per head against a long key/value
cache): the kernel whose four waves share two 64-key blocks per step (one at head_dim 256), through the C ABI, against the
CPU oracle (flash_atten_int8.py:9-66, flash_atten_fp.py:9-60 restated with separate query and key lengths) at the
kernel's 64-key block.

No P requantisation on these paths: kernel and oracle differ by the fp32 summation order inside the MFMA, the hardware
exp2 and where the output is rounded to 16 bits.  Bounds: fp16 max-abs 2e-3 / mean-rel 2e-4, bf16 1.6e-2 / 1.5e-3
(mean-rel = mean|a-b| / mean|b|); LSE 2e-3.
"""
import pytest
import torch

import intfa_oracle as O
import int_flashattention_amd as M

pytestmark = pytest.mark.gpu
DEV = "cuda"


def mean_rel(a, b):
    a, b = a.float().cpu(), b.float().cpu()
    return ((a - b).abs().mean() / b.abs().mean()).item()


def max_abs(a, b):
    return (a.float().cpu() - b.float().cpu()).abs().max().item()


def gpu(*ts):
    return [t.to(DEV) for t in ts]


def bounds(dtype):
    return (2e-3, 2e-4) if dtype == torch.float16 else (1.6e-2, 1.5e-3)


def inputs(B, H, H_kv, Nq, Nk, D, seed, dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((B, H, Nq, D), generator=g).to(dtype)
    k = torch.randn((B, H_kv, Nk, D), generator=g).to(dtype)
    v = torch.randn((B, H_kv, Nk, D), generator=g).to(dtype)
    return q, k, v


def run(variant, q, k, v, causal, sm, **kw):
    if variant == "half":
        q8, qs = O.quant_pertoken(q)
        k8, ks = O.quant_pertoken(k)
        o = M.attention_int8(*gpu(q8, k8, v, qs, ks), causal, sm, **kw)
    else:
        o = M.attention(*gpu(q, k, v), causal, sm, **kw)
    torch.cuda.synchronize()
    return o


def oracle(variant, q, k, v, causal, sm, return_lse=False):
    g = q.shape[1] // k.shape[1]
    rep = lambda t: t.repeat_interleave(g, dim=1)
    bn = M.block_n(variant, q.shape[-1])
    assert bn == 64
    if variant == "half":
        q8, qs = O.quant_pertoken(q)
        k8, ks = O.quant_pertoken(k)
        return O.attention_int8(q8, rep(k8), rep(v), qs, rep(ks), causal, sm, block_n=bn, out_dtype=v.dtype, return_lse=return_lse)
    return O.attention_fp(q, rep(k), rep(v), causal, sm, block_n=bn, return_lse=return_lse)


SHAPES = [
    # B, H, H_kv, Nq, Nk, D, causal
    (2, 4, 4, 1, 1000, 128, False),      # one query per head, ragged cache length
    (1, 8, 2, 1, 2048, 128, False),      # grouped heads: the wrapper folds a group's 4 heads into 4 rows of one head
    (2, 2, 2, 5, 777, 64, False),        # head_dim 64: two of the four waves own an output tile
    (1, 2, 2, 32, 640, 128, False),      # a full 32-row tile, an even number of 64-key blocks
    (1, 2, 2, 33, 577, 128, False),      # two 32-row workgroups per head; an odd number of blocks, the last one ragged
    (1, 2, 1, 7, 50, 128, False),        # cache shorter than one key block
    (1, 2, 2, 2, 1, 64, False),          # a single key
    (1, 2, 2, 64, 64, 64, False),        # exactly one block: the second half of the step is past the end
    (2, 2, 2, 9, 1000, 128, True),       # a few new tokens against a cache (bottom-right aligned mask)
    (1, 8, 2, 6, 333, 64, True),         # grouped heads with the mask: rows carry their position (causal_rows)
    (1, 2, 2, 64, 64, 128, True),        # square: row i sees keys 0 .. i
    (1, 2, 2, 40, 20, 128, True),        # more new tokens than keys: rows above the first key see nothing
    (1, 1, 1, 3, 4096, 128, False),
    # head_dim 256: one 64-key block per step, two output tiles per wave
    (2, 4, 4, 1, 1000, 256, False),
    (1, 8, 2, 1, 2048, 256, False),
    (1, 2, 2, 33, 577, 256, False),
    (1, 2, 1, 7, 50, 256, False),
    (1, 2, 2, 64, 64, 256, True),
    (2, 2, 2, 9, 1000, 256, True),
    (1, 8, 2, 6, 333, 256, True),
    (1, 2, 2, 40, 20, 256, True),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("variant", ["half", "fp"])
@pytest.mark.parametrize("B,H,H_kv,Nq,Nk,D,causal", SHAPES)
def test_decode_matches_oracle(B, H, H_kv, Nq, Nk, D, causal, variant, dtype):
    q, k, v = inputs(B, H, H_kv, Nq, Nk, D, seed=3000 + Nq + Nk, dtype=dtype)
    sm = D ** -0.5
    o, lse = run(variant, q, k, v, causal, sm, return_lse=True)
    assert o.dtype == dtype and o.shape == (B, H, Nq, D) and torch.isfinite(o).all()
    ref, lse_ref = oracle(variant, q, k, v, causal, sm, return_lse=True)
    ma, mr = bounds(dtype)
    assert max_abs(o, ref) <= ma and mean_rel(o, ref) <= mr
    seen = torch.isfinite(lse_ref)
    assert torch.equal(torch.isfinite(lse.cpu()), seen)                    # rows without a key: lse = -inf on both sides
    assert (lse.cpu()[seen] - lse_ref[seen]).abs().max().item() <= 2e-3
    if (~seen).any():
        assert (o.cpu()[~seen] == 0).all()


@pytest.mark.parametrize("variant", ["half", "fp"])
@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("causal", [False, True])
def test_decode_kernel_agrees_with_the_general_kernel(variant, D, causal):
    """65 query rows run the general kernel, 64 of them alone the decode kernel.  At head_dim 256 both take the same block
    maxima, the same 16-bit P and the same MFMA steps per block, so a row's result differs only through the order of the
    fp32 row-sum additions (one rounding of the 16-bit output now and then).  At head_dim <= 128 the general kernel takes
    exp2 against a reference point that lags the running maximum (it rescales the output only when a row's maximum rises by
    more than 8), the decode kernel against the running maximum itself as the oracle does: the same p up to a factor that
    cancels in acc / l, rounded to 16 bits at another place (relative 2^-12 per element, unbiased) - a few 1e-4 in the mean.
    With the mask the 64 rows are the LAST 64 of the 65 (the mask is aligned to the end of the cache)."""
    q, k, v = inputs(1, 2, 2, 65, 1500, D, seed=3100 + D)
    sm = D ** -0.5
    general, lg = run(variant, q, k, v, causal, sm, return_lse=True)
    rows = slice(1, 65) if causal else slice(0, 64)
    decode, ld = run(variant, q[:, :, rows].contiguous(), k, v, causal, sm, return_lse=True)
    assert max_abs(decode, general[:, :, rows]) <= 1e-3 and mean_rel(decode, general[:, :, rows]) <= (2e-5 if D == 256 else 6e-4)
    assert (ld - lg[:, :, rows]).abs().max().item() <= 1e-4


@pytest.mark.parametrize("variant", ["half", "fp"])
@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("Nq,Nk,causal,splits", [(3, 2000, False, 2), (3, 2000, False, 5), (1, 4100, False, "auto"), (17, 1000, True, 3),
                                                 (40, 333, True, 4)])
def test_decode_split_kv_equals_single_pass(variant, D, Nq, Nk, causal, splits):
    """The split evaluation is the same sum in another order, except that P is cast to 16 bits relative to another running
    maximum: it agrees with the single pass to a fraction of an output ulp in the mean, and its LSE to fp32 rounding."""
    q, k, v = inputs(2, 4, 4, Nq, Nk, D, seed=3200 + Nq)
    sm = D ** -0.5
    o1, l1 = run(variant, q, k, v, causal, sm, return_lse=True)
    o2, l2 = run(variant, q, k, v, causal, sm, num_splits=splits, return_lse=True)
    assert torch.isfinite(o2).all()
    assert max_abs(o2, o1) <= 1e-3 and mean_rel(o2, o1) <= 5e-4
    assert (l1 - l2).abs().max().item() <= 1e-3
    ref = oracle(variant, q, k, v, causal, sm)
    assert max_abs(o2, ref) <= 2e-3 and mean_rel(o2, ref) <= 3e-4


@pytest.mark.parametrize("variant", ["half", "fp"])
@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("causal", [False, True])
def test_decode_per_batch_cache_lengths(variant, D, causal):
    """seqlens_k: every batch entry comes out as a call on that entry with the cache cut to its length (an empty entry
    gives zeros)."""
    B, H, Nq, Nk = 4, 2, 5, 600
    lens = [600, 1, 333, 0]
    q, k, v = inputs(B, H, H, Nq, Nk, D, seed=3300)
    sm = D ** -0.5
    o = run(variant, q, k, v, causal, sm, seqlens_k=torch.tensor(lens, dtype=torch.int32, device=DEV))
    for b, n in enumerate(lens):
        if n == 0:
            assert (o[b] == 0).all()
            continue
        ob = run(variant, q[b:b + 1], k[b:b + 1, :, :n], v[b:b + 1, :, :n], causal, sm)
        assert torch.equal(o[b:b + 1], ob), (b, n)


@pytest.mark.parametrize("variant", ["half", "fp"])
@pytest.mark.parametrize("causal", [False, True])
def test_decode_grouped_heads_equal_repeated_kv(variant, causal):
    """The fold of a group's query heads into rows of one head changes which rows share a workgroup, nothing else."""
    B, H, H_kv, Nq, Nk, D = 2, 8, 2, 4, 700, 128
    q, k, v = inputs(B, H, H_kv, Nq, Nk, D, seed=3400)
    sm = D ** -0.5
    o = run(variant, q, k, v, causal, sm)
    rep = lambda t: t.repeat_interleave(H // H_kv, dim=1)
    o_rep = run(variant, q, rep(k), rep(v), causal, sm)
    assert torch.equal(o, o_rep)
    ref = oracle(variant, q, k, v, causal, sm)
    assert max_abs(o, ref) <= 2e-3 and mean_rel(o, ref) <= 2e-4


@pytest.mark.parametrize("variant", ["half", "fp"])
def test_decode_strided_cache_and_guard_region(variant):
    """The cache lives in a longer allocation with padded rows; nothing is written behind the output rows."""
    B, H, Nq, Nk, D = 2, 2, 3, 500, 128
    q, k, v = inputs(B, H, H, Nq, Nk, D, seed=3500)
    sm = D ** -0.5
    big = lambda t: torch.cat([t, torch.zeros_like(t[:, :, :100])], dim=2)[:, :, :Nk]       # batch / head strides of 600 rows
    if variant == "half":
        q8, qs = O.quant_pertoken(q)
        k8, ks = O.quant_pertoken(k)
        a = gpu(q8, k8, v, qs, ks)
        a[1], a[2] = big(a[1]), big(a[2])
        assert not a[1].is_contiguous()
        o = M.attention_int8(*a, False, sm)
    else:
        a = gpu(q, k, v)
        a[1], a[2] = big(a[1]), big(a[2])
        o = M.attention(*a, False, sm)
    torch.cuda.synchronize()
    ref = oracle(variant, q, k, v, False, sm)
    assert max_abs(o, ref) <= 2e-3 and mean_rel(o, ref) <= 2e-4


@pytest.mark.parametrize("variant", ["half", "fp"])
def test_decode_full_size_against_one_head_of_the_oracle(variant):
    """B32 H32 Nk4096 d128, one query per head (a bench workload of these kernels): reproducible between two launches,
    three (batch, head) slices against the oracle."""
    B, H, Nk, D = 32, 32, 4096, 128
    g = torch.Generator(device=DEV).manual_seed(3600)
    q = torch.randn((B, H, 1, D), generator=g, device=DEV).half()
    k = torch.randn((B, H, Nk, D), generator=g, device=DEV).half()
    v = torch.randn((B, H, Nk, D), generator=g, device=DEV).half()
    sm = D ** -0.5
    if variant == "half":
        q8, qs = M.quant_pertoken(q)
        k8, ks = M.quant_pertoken(k)
        call = lambda: M.attention_int8(q8, k8, v, qs, ks, False, sm)
    else:
        call = lambda: M.attention(q, k, v, False, sm)
    o1, o2 = call(), call()
    torch.cuda.synchronize()
    assert torch.equal(o1, o2) and torch.isfinite(o1).all()
    for b, h in ((0, 0), (31, 31), (13, 7)):
        c = lambda t: t[b:b + 1, h:h + 1].cpu()
        if variant == "half":
            ref = O.attention_int8(c(q8), c(k8), c(v), c(qs), c(ks), False, sm, block_n=64)
        else:
            ref = O.attention_fp(c(q), c(k), c(v), False, sm, block_n=64)
        assert max_abs(o1[b:b + 1, h:h + 1], ref) <= 2e-3 and mean_rel(o1[b:b + 1, h:h + 1], ref) <= 2e-4, (b, h)
