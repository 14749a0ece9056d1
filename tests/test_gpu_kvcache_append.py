"""GPU parity of the append to an int8 K/V cache (intfa_kvcache_append_int8) through the C ABI: bit for bit against the
CPU oracle, and end to end: a cache built by appends, read by the decode forward with per-batch lengths, gives what the
forward gives on the directly quantised concatenation."""
import pytest
import torch

import intfa_oracle as O
import int_flashattention_amd as M
from test_gpu_parity import DEV

pytestmark = pytest.mark.gpu


def _caches(Z, H, n_cache, d, dtype):
    g = torch.Generator().manual_seed(3)
    kc = torch.randint(-128, 128, (Z, H, n_cache, d), generator=g, dtype=torch.int8)
    vc = torch.randint(-128, 128, (Z, H, n_cache, d), generator=g, dtype=torch.int8)
    ksc = torch.rand((Z, H, n_cache), generator=g).to(dtype)
    return kc, vc, ksc


@pytest.mark.parametrize("Z,H,n_new,n_cache,d,dtype,lens", [
    (2, 3, 1, 64, 128, torch.float16, [0, 63]),          # one token per entry, the second into the last slot
    (3, 2, 5, 40, 64, torch.bfloat16, [0, 17, 38]),      # the third entry has room for two of its five rows
    (1, 4, 33, 200, 256, torch.float16, [100]),
    (2, 1, 7, 30, 16, torch.bfloat16, [30, 3]),          # a full cache takes nothing
    (2, 2, 4, 50, 32, torch.float16, 9),                 # one length for all entries
])
def test_append_is_bit_exact(Z, H, n_new, n_cache, d, dtype, lens):
    g = torch.Generator().manual_seed(11)
    k_new = torch.randn((Z, H, n_new, d), generator=g).to(dtype)
    v_new = (torch.randn((Z, H, n_new, d), generator=g) * 2).to(dtype)      # some values beyond the cache's V scale
    vs = (torch.rand((Z, H), generator=g) * 0.02 + 0.01).to(dtype)
    kc, vc, ksc = _caches(Z, H, n_cache, d, dtype)
    kc_ref, vc_ref, ksc_ref = kc.clone(), vc.clone(), ksc.clone()
    lens_list = [lens] * Z if isinstance(lens, int) else lens
    O.kvcache_append(kc_ref, ksc_ref, k_new, lens_list, vc_ref, vs, v_new)
    kc_d, vc_d, ksc_d = kc.to(DEV), vc.to(DEV), ksc.to(DEV)
    lens_d = lens if isinstance(lens, int) else torch.tensor(lens, dtype=torch.int32, device=DEV)
    M.kvcache_append(kc_d, ksc_d, k_new.to(DEV), lens_d, vc_d, vs.to(DEV), v_new.to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(kc_d.cpu(), kc_ref) and torch.equal(vc_d.cpu(), vc_ref)
    assert torch.equal(ksc_d.cpu().view(torch.int16), ksc_ref.view(torch.int16))
    assert (vc_ref.abs() == 127).any()                                       # the saturation was exercised


def test_append_keys_only_and_strided_new_tokens():
    """K alone (the half-int8 variant keeps V in 16 bits), new tokens handed over as a [Z, N, H, d] view."""
    Z, H, n_new, n_cache, d = 2, 4, 3, 20, 64
    g = torch.Generator().manual_seed(12)
    k_new = torch.randn((Z, n_new, H, d), generator=g).half().permute(0, 2, 1, 3)       # strides of a bshd tensor
    kc, vc, ksc = _caches(Z, H, n_cache, d, torch.float16)
    kc_ref, ksc_ref = kc.clone(), ksc.clone()
    O.kvcache_append(kc_ref, ksc_ref, k_new, [5, 0])
    kc_d, ksc_d = kc.to(DEV), ksc.to(DEV)
    M.kvcache_append(kc_d, ksc_d, k_new.to(DEV), torch.tensor([5, 0], dtype=torch.int32, device=DEV))
    torch.cuda.synchronize()
    assert torch.equal(kc_d.cpu(), kc_ref) and torch.equal(ksc_d.cpu(), ksc_ref)


def test_cache_built_by_appends_decodes_like_the_quantised_concatenation():
    """Prefill of different lengths per entry, then two decode steps: append the step's key/value, attend with one query
    per head over the entry's filled length.  The appended cache holds exactly the int8 rows and scales of quantising the
    whole sequence at once (V with the same per-(batch, head) scale), so the outputs must be identical."""
    Z, H, H_kv, d, n_cache = 2, 8, 2, 128, 384
    g = torch.Generator().manual_seed(13)
    lens = [200, 317]
    k = torch.randn((Z, H_kv, n_cache, d), generator=g).half(); v = torch.randn((Z, H_kv, n_cache, d), generator=g).half()
    _, vs = O.quant_pertensor(v)                                               # the cache's V scale, fixed up front
    kc = torch.zeros((Z, H_kv, n_cache, d), dtype=torch.int8, device=DEV); vc = torch.zeros_like(kc)
    ksc = torch.zeros((Z, H_kv, n_cache), dtype=torch.float16, device=DEV)
    vs_d = vs.to(DEV)
    zero = torch.zeros((Z,), dtype=torch.int32, device=DEV)
    for b in range(Z):                                                          # prefill entry b alone (lengths differ)
        M.kvcache_append(kc[b:b + 1], ksc[b:b + 1], k[b:b + 1, :, :lens[b]].to(DEV), zero[:1], vc[b:b + 1], vs_d[b:b + 1],
                         v[b:b + 1, :, :lens[b]].to(DEV))
    lens_d = torch.tensor(lens, dtype=torch.int32, device=DEV)
    sm = d ** -0.5
    for step in range(2):
        k_new = torch.stack([k[b, :, lens[b] + step:lens[b] + step + 1] for b in range(Z)])
        v_new = torch.stack([v[b, :, lens[b] + step:lens[b] + step + 1] for b in range(Z)])
        M.kvcache_append(kc, ksc, k_new.to(DEV), lens_d, vc, vs_d, v_new.to(DEV))
        lens_d = lens_d + 1
        q = torch.randn((Z, H, 1, d), generator=g).half()
        q8, qs = M.quant_pertoken(q.to(DEV))
        o = M.attention_full_int8(q8, kc, vc, qs, ksc, vs_d, False, sm, seqlens_k=lens_d, p_round="rne")
        for b in range(Z):
            n = lens[b] + step + 1
            k8, ks = M.quant_pertoken(k[b:b + 1, :, :n].to(DEV))
            v8 = torch.round(v[b:b + 1, :, :n] / vs[b:b + 1, :, None, None]).clamp(-127, 127).to(torch.int8).to(DEV)
            want = M.attention_full_int8(q8[b:b + 1], k8, v8, qs[b:b + 1], ks, vs_d[b:b + 1], False, sm, p_round="rne")
            assert torch.equal(o[b:b + 1], want)
