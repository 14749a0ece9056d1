"""Half-int8 and fp16/bf16 attention at head_dim 256: the eight-wave kernel in which two waves share 32 query rows
(each computes the softmax of half of a 64-key block and the output of half of the columns).

No P requantisation on these paths: against the oracle (flash_atten_int8.py:9-66, flash_atten_fp.py:9-60 restated with
the kernel's 64-key block) the only differences are the fp32 summation order inside the MFMA, the hardware exp2 and where
the output is rounded to 16 bits, so the bounds are a few output ulps: fp16 max-abs 2e-3 / mean-rel 2e-4, bf16 1.6e-2 /
1.5e-3 (mean-rel = mean|a-b| / mean|b|).
"""
import pytest
import torch

import intfa_oracle as O
import int_flashattention_amd as M

pytestmark = pytest.mark.gpu
DEV = "cuda"
D = 256


def mean_rel(a, b):
    a, b = a.float().cpu(), b.float().cpu()
    return ((a - b).abs().mean() / b.abs().mean()).item()


def max_abs(a, b):
    return (a.float().cpu() - b.float().cpu()).abs().max().item()


def gpu(*ts):
    return [t.to(DEV) for t in ts]


def bounds(dtype):
    return (2e-3, 2e-4) if dtype == torch.float16 else (1.6e-2, 1.5e-3)


def inputs(B, H, Nq, Nk, seed, dtype=torch.float16, H_kv=None):
    g = torch.Generator().manual_seed(seed)
    H_kv = H if H_kv is None else H_kv
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
    bn = M.block_n(variant, D)
    assert bn == 64
    if variant == "half":
        q8, qs = O.quant_pertoken(q)
        k8, ks = O.quant_pertoken(k)
        return O.attention_int8(q8, k8, v, qs, ks, causal, sm, block_n=bn, out_dtype=v.dtype, return_lse=return_lse)
    return O.attention_fp(q, k, v, causal, sm, block_n=bn, return_lse=return_lse)


def repeat_kv(t, g):
    return t.repeat_interleave(g, dim=1)


SHAPES = [
    # B, H, Nq, Nk, causal
    (1, 2, 128, 128, False),      # one query block, two key blocks
    (2, 3, 384, 384, True),       # paired query blocks (one left over), diagonal blocks
    (1, 2, 512, 512, True),       # paired query blocks, even count
    (1, 2, 300, 300, False),      # ragged rows and keys
    (1, 2, 641, 641, True),
    (1, 2, 1, 700, False),        # one query row against a cache
    (2, 2, 37, 1000, True),       # a few new tokens against a cache (bottom-right aligned mask)
    (1, 2, 200, 77, False),       # more queries than keys
    (1, 2, 200, 77, True),        # rows above the first key see nothing
    (1, 1, 130, 2048, False),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("variant", ["half", "fp"])
@pytest.mark.parametrize("B,H,Nq,Nk,causal", SHAPES)
def test_matches_oracle(B, H, Nq, Nk, causal, variant, dtype):
    q, k, v = inputs(B, H, Nq, Nk, seed=2560 + Nq + Nk, dtype=dtype)
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
@pytest.mark.parametrize("Nq,Nk,causal,splits", [(256, 1024, False, 2), (256, 1024, True, 3), (384, 384, True, 5), (1, 2000, False, 4),
                                                 (511, 511, True, 3)])
def test_split_kv_equals_single_pass(variant, Nq, Nk, causal, splits):
    """The split evaluation is the same sum in another order, except that P is cast to 16 bits relative to another running
    maximum: it agrees with the single pass to a fraction of an output ulp in the mean, and its LSE to fp32 rounding."""
    q, k, v = inputs(1, 2, Nq, Nk, seed=2570 + splits)
    sm = D ** -0.5
    o1, l1 = run(variant, q, k, v, causal, sm, return_lse=True)
    o2, l2 = run(variant, q, k, v, causal, sm, num_splits=splits, return_lse=True)
    assert torch.isfinite(o2).all()
    assert max_abs(o2, o1) <= 1e-3 and mean_rel(o2, o1) <= 5e-4
    assert (l1 - l2).abs().max().item() <= 1e-3
    ref = oracle(variant, q, k, v, causal, sm)
    assert max_abs(o2, ref) <= 2e-3 and mean_rel(o2, ref) <= 3e-4


@pytest.mark.parametrize("variant", ["half", "fp"])
@pytest.mark.parametrize("causal", [False, True])
def test_grouped_heads_equal_repeated_kv(variant, causal):
    B, H, H_kv, N = 2, 8, 2, 256
    q, k, v = inputs(B, H, N, N, seed=2580, H_kv=H_kv)
    sm = D ** -0.5
    o = run(variant, q, k, v, causal, sm)
    o_rep = run(variant, q, repeat_kv(k, H // H_kv), repeat_kv(v, H // H_kv), causal, sm)
    assert torch.equal(o, o_rep)                                            # the same arithmetic on the same numbers
    ref = oracle(variant, q, repeat_kv(k, H // H_kv), repeat_kv(v, H // H_kv), causal, sm)
    assert max_abs(o, ref) <= 2e-3 and mean_rel(o, ref) <= 2e-4


@pytest.mark.parametrize("variant", ["half", "fp"])
@pytest.mark.parametrize("causal", [False, True])
def test_per_batch_cache_lengths(variant, causal):
    """seqlens_k: every batch entry comes out as a call on that entry with the cache cut to its length."""
    B, H, Nq, Nk = 3, 2, 40, 600
    lens = [600, 1, 333]
    q, k, v = inputs(B, H, Nq, Nk, seed=2590)
    sm = D ** -0.5
    o = run(variant, q, k, v, causal, sm, seqlens_k=torch.tensor(lens, dtype=torch.int32, device=DEV))
    for b, n in enumerate(lens):
        ob = run(variant, q[b:b + 1], k[b:b + 1, :, :n], v[b:b + 1, :, :n], causal, sm)
        assert torch.equal(o[b:b + 1], ob), (b, n)


@pytest.mark.parametrize("variant", ["half", "fp"])
def test_strided_inputs_and_guard_region(variant):
    """Inputs that are views with padded rows; nothing is written behind the output rows of a ragged problem."""
    B, H, N = 1, 2, 200
    q, k, v = inputs(B, H, N, N, seed=2600)
    pad = lambda t: torch.cat([t, torch.full_like(t[..., :16], 7)], dim=-1)[..., :D]      # row stride D + 16
    sm = D ** -0.5
    if variant == "half":
        q8, qs = O.quant_pertoken(q)
        k8, ks = O.quant_pertoken(k)
        a = gpu(q8, k8, v, qs, ks)
        a[0], a[1], a[2] = pad(a[0]), pad(a[1]), pad(a[2])
        o = M.attention_int8(*a, True, sm)
    else:
        a = [pad(t) for t in gpu(q, k, v)]
        o = M.attention(*a, True, sm)
    torch.cuda.synchronize()
    assert not a[0].is_contiguous()
    ref = oracle(variant, q, k, v, True, sm)
    assert max_abs(o, ref) <= 2e-3 and mean_rel(o, ref) <= 2e-4


@pytest.mark.parametrize("variant", ["half", "fp"])
def test_benchmark_sized_slice(variant):
    """B4 H32 N4096 d256 (the bench workloads of these kernels): three (batch, head) slices against the oracle."""
    B, H, N = 4, 32, 4096
    g = torch.Generator(device=DEV).manual_seed(2610)
    mk = lambda: torch.randn((B, H, N, D), generator=g, device=DEV, dtype=torch.float32).half()
    q, k, v = mk(), mk(), mk()
    sm = D ** -0.5
    if variant == "half":
        q8, qs = M.quant_pertoken(q)
        k8, ks = M.quant_pertoken(k)
        o = M.attention_int8(q8, k8, v, qs, ks, False, sm)
    else:
        o = M.attention(q, k, v, False, sm)
    torch.cuda.synchronize()
    assert torch.isfinite(o).all()
    for b, h in ((0, 0), (3, 31), (1, 17)):
        c = lambda t: t[b:b + 1, h:h + 1].cpu()
        if variant == "half":
            ref = O.attention_int8(c(q8), c(k8), c(v), c(qs), c(ks), False, sm, block_n=64)
        else:
            ref = O.attention_fp(c(q), c(k), c(v), False, sm, block_n=64)
        assert max_abs(o[b:b + 1, h:h + 1], ref) <= 2e-3 and mean_rel(o[b:b + 1, h:h + 1], ref) <= 2e-4, (b, h)
