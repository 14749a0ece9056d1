"""Tensors whose batch entries lie more than 2^31 and 2^32 bytes apart: the kernels add batch and head strides in 64 bits
(only the offset inside one (batch, head) slice is 32-bit, and the entry points reject slices of 4 GiB and more).

Each operand is a strided view into a large flat buffer (batch stride 2.3 GiB for the 8-bit tensors, 1.2 G elements for
the 16-bit ones), so only a few MiB are touched.  The result must equal, bit for bit, the result of the same call on
contiguous copies: the arithmetic does not depend on where the rows lie.
"""
import pytest
import torch

import intfa_oracle as O
import int_flashattention_amd as M

pytestmark = pytest.mark.gpu
DEV = "cuda"
FAR = 2_300_000_000 + 1024          # elements between batch entries (a multiple of 16 bytes for every element size used)


@pytest.fixture(autouse=True)
def _release_buffers():
    yield
    torch.cuda.empty_cache()            # each case holds tens of GiB of (untouched) address space


def far_view(t):
    """A copy of t ([B, H, N, d] or [B, H, N] or [B, H]) whose batch entries lie FAR elements apart."""
    B = t.shape[0]
    inner = t[0].numel()
    buf = torch.empty(FAR * (B - 1) + inner, dtype=t.dtype, device=t.device)
    strides = (FAR,) + tuple(t[0].contiguous().stride())
    v = torch.as_strided(buf, t.shape, strides)
    v.copy_(t)
    return v


def quantised(B, H, Hkv, Nq, Nk, D, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((B, H, Nq, D), generator=g).half()
    k = torch.randn((B, Hkv, Nk, D), generator=g).half()
    v = torch.randn((B, Hkv, Nk, D), generator=g).half()
    q8, qs = O.quant_pertoken(q)
    k8, ks = O.quant_pertoken(k)
    v8, vs = O.quant_pertensor(v)
    return [t.to(DEV) for t in (q, k, v, q8, qs, k8, ks, v8, vs)]


@pytest.mark.parametrize("Nq,Nk,D,causal,splits", [(512, 512, 128, True, 1), (300, 700, 64, False, 2), (1, 2048, 128, False, 1),
                                                  (16, 1500, 256, True, 2), (256, 256, 256, False, 1)])
def test_full_int8_batch_entries_far_apart(Nq, Nk, D, causal, splits):
    B, H, Hkv = 3, 4, 2
    q, k, v, q8, qs, k8, ks, v8, vs = quantised(B, H, Hkv, Nq, Nk, D, 77)
    sm = D ** -0.5
    want, lse_w = M.attention_full_int8(q8, k8, v8, qs, ks, vs, causal, sm, num_splits=splits, return_lse=True, p_round="rne")
    got, lse_g = M.attention_full_int8(far_view(q8), far_view(k8), far_view(v8), far_view(qs), far_view(ks), far_view(vs), causal, sm,
                                       num_splits=splits, return_lse=True, p_round="rne")
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(lse_g, lse_w)
    assert bool(torch.isfinite(got).all()) and got.abs().max().item() > 0


@pytest.mark.parametrize("Nq,Nk,D,causal,splits", [(512, 512, 128, True, 1), (300, 700, 64, False, 2), (1, 2048, 128, False, 1),
                                                  (16, 1500, 256, True, 1), (384, 384, 256, False, 2)])
def test_half_int8_and_fp_batch_entries_far_apart(Nq, Nk, D, causal, splits):
    B, H, Hkv = 3, 4, 2
    q, k, v, q8, qs, k8, ks, v8, vs = quantised(B, H, Hkv, Nq, Nk, D, 78)
    sm = D ** -0.5
    want = M.attention_int8(q8, k8, v, qs, ks, causal, sm, num_splits=splits)
    got = M.attention_int8(far_view(q8), far_view(k8), far_view(v), far_view(qs), far_view(ks), causal, sm, num_splits=splits)
    assert torch.equal(got, want) and got.abs().max().item() > 0
    want = M.attention(q, k, v, causal, sm, num_splits=splits)
    got = M.attention(far_view(q), far_view(k), far_view(v), causal, sm, num_splits=splits)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and got.abs().max().item() > 0


def test_quantisers_and_cache_append_rows_far_apart():
    B, H, N, D = 3, 2, 256, 128
    g = torch.Generator().manual_seed(79)
    x = torch.randn((B, H, N, D), generator=g).half().to(DEV)
    q_want, s_want = M.quant_pertoken(x)
    q_got, s_got = M.quant_pertoken(far_view(x))
    assert torch.equal(q_got, q_want) and torch.equal(s_got, s_want)
    q_want, s_want = M.quant_pertensor(x)
    q_got, s_got = M.quant_pertensor(far_view(x))
    torch.cuda.synchronize()
    assert torch.equal(q_got, q_want) and torch.equal(s_got, s_want)


def test_cache_append_into_a_cache_whose_entries_lie_far_apart():
    Z, H, n_new, n_cache, d = 3, 2, 5, 64, 128
    g = torch.Generator().manual_seed(80)
    k_new = torch.randn((Z, H, n_new, d), generator=g).half().to(DEV)
    v_new = torch.randn((Z, H, n_new, d), generator=g).half().to(DEV)
    vs = (torch.rand((Z, H), generator=g) * 0.02 + 0.02).half().to(DEV)
    lens = torch.tensor([7, 0, 59], dtype=torch.int32, device=DEV)
    kc = torch.zeros((Z, H, n_cache, d), dtype=torch.int8, device=DEV)
    vc = torch.zeros_like(kc)
    ksc = torch.zeros((Z, H, n_cache), dtype=torch.float16, device=DEV)
    kc_f, vc_f, ksc_f = far_view(kc), far_view(vc), far_view(ksc)
    M.kvcache_append(kc, ksc, k_new, lens, vc, vs, v_new)
    M.kvcache_append(kc_f, ksc_f, far_view(k_new), lens, vc_f, far_view(vs), far_view(v_new))
    torch.cuda.synchronize()
    assert torch.equal(kc_f, kc) and torch.equal(vc_f, vc) and torch.equal(ksc_f, ksc)
    assert kc.abs().max().item() == 127
