"""Pins the CPU oracle (oracle/intfa_oracle.py) by means that do not retype its formulas: closed forms,
invariants, special cases that reduce to library routines, and brute force on tiny inputs.

The reference holds no golden vectors for the int8 paths (its single test asserts the fp16 forward with
atol=1e-2, benchmark.py:242); that tolerance is used for the fp16 oracle below.
"""
import math

import numpy as np
import pytest
import torch

import intfa_oracle as O


# ------------------------------------------------------------------------------------------ quantisers
def test_quant_pertoken_invariants_and_bruteforce():
    g = torch.Generator().manual_seed(0)
    x = torch.randn((2, 3, 5, 16), generator=g).half()
    q, s = O.quant_pertoken(x)
    assert q.dtype == torch.int8 and s.shape == (2, 3, 5) and s.dtype == torch.float16
    assert int(q.abs().max()) == 127                      # every row reaches +-127
    assert torch.all(q.abs().amax(dim=-1) == 127)
    xn, sn = x.numpy(), s.numpy()
    for idx in np.ndindex(2, 3, 5):                       # scalar restatement in numpy float16 arithmetic
        row = xn[idx]
        sc = np.float16(np.abs(row).max()) / np.float16(127)
        assert sc == sn[idx]
        for j in range(16):
            want = int(np.rint(np.float16(row[j] / sc)))  # np.rint rounds half to even
            assert want == int(q[idx][j])


def test_quant_pertensor_one_scale_per_head():
    g = torch.Generator().manual_seed(1)
    x = torch.randn((2, 2, 8, 4), generator=g).half()
    q, s = O.quant_pertensor(x)
    assert s.shape == (2, 2)
    for b in range(2):
        for h in range(2):
            assert float(s[b, h]) == float((x[b, h].abs().max() / 127))
            assert int(q[b, h].abs().max()) == 127


def test_mean_relative_error_matches_reference_definition():
    a = torch.tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0])
    b = torch.tensor([1.0, 2.0, 3.3, 4.0, 5.0, 6.6])
    # the reference looks at the last four elements only: |b-a| / (|b| + 1e-5)
    want = np.mean([abs(3.3 - 3.0) / (3.3 + 1e-5), 0.0, 0.0, abs(6.6 - 6.0) / (6.6 + 1e-5)])
    assert abs(O.mean_relative_error(a, b, calc_num=4) - want) < 1e-6
    assert O.mean_relative_error(a, a) == 0.0


# ------------------------------------------------------------------------------------------ integer parts
def test_qk_int32_is_exact_integer_matmul():
    g = torch.Generator().manual_seed(2)
    q8 = torch.randint(-127, 128, (1, 2, 6, 8), generator=g, dtype=torch.int8)
    k8 = torch.randint(-127, 128, (1, 2, 6, 8), generator=g, dtype=torch.int8)
    s = O.qk_int32(q8, k8)
    assert s.dtype == torch.int32
    for h in range(2):
        for i in range(6):
            for j in range(6):
                want = sum(int(q8[0, h, i, t]) * int(k8[0, h, j, t]) for t in range(8))
                assert int(s[0, h, i, j]) == want
    # extreme values at the largest head dim: |S| = 127*127*256 must survive the fp32 GEMM exactly
    q8 = torch.full((1, 1, 2, 256), 127, dtype=torch.int8)
    k8 = torch.full((1, 1, 2, 256), -127, dtype=torch.int8)
    assert torch.all(O.qk_int32(q8, k8) == -127 * 127 * 256)
    big = np.random.default_rng(0).integers(-127, 128, size=(2, 64, 256))
    got = O.qk_int32(torch.tensor(big[None, :1], dtype=torch.int8), torch.tensor(big[None, 1:], dtype=torch.int8))
    assert np.array_equal(got[0, 0].numpy().astype(np.int64), big[0].astype(np.int64) @ big[1].astype(np.int64).T)


def test_p_requant_reference_exhaustive_over_fp16():
    """Every fp16 value in [0, 1]: fp16(p)*127 -> fp16, +0.5 -> fp16, truncate (flash_atten_full_int8.py:49-51)."""
    bits = np.arange(0, 0x3C01, dtype=np.uint16)          # 0.0 .. 1.0 inclusive
    p = bits.view(np.float16)
    got = O.p_requant_reference(torch.from_numpy(p.astype(np.float32))).numpy()
    w = (p * np.float16(127)).astype(np.float16)           # numpy rounds each fp16 operation to fp16
    u = (w + np.float16(0.5)).astype(np.float16)
    want = np.trunc(u.astype(np.float32))
    assert np.array_equal(got, want)
    assert got.min() == 0 and got.max() == 127
    # values between fp16 grid points are first rounded to fp16 (round-to-nearest-even)
    x = torch.tensor([0.50006, 0.1234567, 0.99999, 1e-9])
    got = O.p_requant_reference(x).numpy()
    for v, gq in zip(x.numpy(), got):
        hv = np.float16(v)
        assert gq == np.trunc(np.float32(np.float16(np.float16(hv * np.float16(127)) + np.float16(0.5))))


def test_p_requant_rne_is_round_half_even_of_127p():
    """The kernels' default rounding: 127*p in fp32, rounded to nearest-even, saturating at 255."""
    p = np.concatenate([np.linspace(0, 1, 200001, dtype=np.float32), (np.arange(0, 128, dtype=np.float32) + 0.5) / 127])
    got = O.p_requant_rne(torch.from_numpy(p)).numpy()
    want = np.clip(np.rint(p * np.float32(127.0)), 0, 255)
    assert np.array_equal(got, want)
    assert O.p_requant_rne(torch.tensor([2.5 / 127, 3.5 / 127])).tolist() == [np.rint(np.float32(2.5 / 127) * np.float32(127)),
                                                                                np.rint(np.float32(3.5 / 127) * np.float32(127))]
    assert O.p_requant_rne(torch.tensor([3.0])).item() == 255


def test_p_requant_modes_differ_by_at_most_one():
    p = torch.linspace(0, 1, 100001)
    d = (O.p_requant_reference(p) - O.p_requant_rne(p)).abs()
    assert d.max() <= 1


# ------------------------------------------------------------------------------------------ online softmax
def _dense_attention(x, v, causal):
    """softmax over keys of logits x (already scaled, natural-log domain) times v, all fp32, torch.softmax."""
    if causal:
        n = x.shape[-1]
        x = x.masked_fill(~torch.tril(torch.ones((n, n), dtype=torch.bool)), float("-inf"))
    return torch.softmax(x, dim=-1) @ v


@pytest.mark.parametrize("causal", [False, True])
def test_fp_variant_reduces_to_torch_softmax_for_any_block(causal):
    q, k, v, _ = O.make_inputs(1, 2, 64, 16, seed=3, std=0.5)
    sm = 0.3
    want = _dense_attention((q.float() @ k.float().transpose(2, 3)) * sm, v.float(), causal)
    for bm, bn in ((64, 64), (32, 16), (16, 16), (64, 8)):
        got, lse = O.attention_fp(q, k, v, causal, sm, block_m=bm, block_n=bn, return_lse=True)
        # P is rounded to fp16 before PV (flash_atten_fp.py:54); the reference's own tolerance is atol=1e-2
        assert (got.float() - want).abs().max() < 2e-3
        x = (q.float() @ k.float().transpose(2, 3)) * sm
        if causal:
            x = x.masked_fill(~torch.tril(torch.ones((64, 64), dtype=torch.bool)), float("-inf"))
        want_lse = torch.logsumexp(x, dim=-1) * O.LOG2E      # M = m + log2(l) is the base-2 log-sum-exp
        assert (lse - want_lse).abs().max() < 1e-4


def test_half_variant_dense_special_case():
    """Half-int8 with block_n = N is dequantise -> torch.softmax -> fp16(P) @ V."""
    q, k, v, _ = O.make_inputs(1, 2, 32, 16, seed=4)
    q8, qs = O.quant_pertoken(q)
    k8, ks = O.quant_pertoken(k)
    sm = 0.25
    x = (q8.float() @ k8.float().transpose(2, 3)) * qs.float()[..., None] * ks.float()[:, :, None, :]
    pm = torch.softmax(x * sm, dim=-1)
    got = O.attention_int8(q8, k8, v, qs, ks, False, sm, block_m=32, block_n=32)
    # oracle rounds the UNNORMALISED p (<= 1) to fp16 and divides by l afterwards
    want = pm @ v.float()
    assert (got.float() - want).abs().max() < 2e-3
    for bn in (8, 16):
        other = O.attention_int8(q8, k8, v, qs, ks, False, sm, block_m=32, block_n=bn)
        assert (other.float() - got.float()).abs().max() < 2e-3


def test_full_int8_unit_scales_is_integer_attention_bruteforce():
    """All scales one, tiny integers: evaluate the reference loop with Python scalars for one head."""
    g = torch.Generator().manual_seed(5)
    N, D, BN = 4, 2, 2
    q8 = torch.randint(-3, 4, (1, 1, N, D), generator=g, dtype=torch.int8)
    k8 = torch.randint(-3, 4, (1, 1, N, D), generator=g, dtype=torch.int8)
    v8 = torch.randint(-127, 128, (1, 1, N, D), generator=g, dtype=torch.int8)
    one = torch.ones((1, 1, N), dtype=torch.float16)
    vs = torch.ones((1, 1), dtype=torch.float16)
    sm = 0.5
    got = O.attention_full_int8(q8, k8, v8, one, one, vs, False, sm, block_m=2, block_n=BN).float()[0, 0]
    c = np.float32(sm) * np.float32(O.LOG2E)
    for i in range(N):
        m, l, acc = -math.inf, 1.0, [0.0] * D
        for j0 in range(0, N, BN):
            s = [sum(int(q8[0, 0, i, t]) * int(k8[0, 0, j, t]) for t in range(D)) for j in range(j0, j0 + BN)]
            m_new = max(m, max(np.float32(x) * c for x in s))
            p = [float(np.exp2(np.float32(np.float32(x) * c - np.float32(m_new)))) for x in s]
            p8 = [int(np.trunc(np.float32(np.float16(np.float16(np.float16(x) * np.float16(127)) + np.float16(0.5))))) for x in p]
            alpha = float(np.exp2(np.float32(m - m_new))) if m != -math.inf else 0.0
            l = l * alpha + sum(p)
            for t in range(D):
                tmp = sum(p8[jj] * int(v8[0, 0, j0 + jj, t]) for jj in range(BN))
                acc[t] = acc[t] * alpha + tmp * 1.0 / 127
            m = m_new
        for t in range(D):
            assert abs(got[i, t].item() - acc[t] / l) <= 1e-3 * max(1.0, abs(acc[t] / l))


def test_full_int8_constant_v_gives_quantised_mass_ratio():
    """V8 == c everywhere: O = c * v_scale * sum(P8) / (127 * l); with one key block sum(P8) and l are dense."""
    q, k, _, _ = O.make_inputs(1, 1, 16, 8, seed=6)
    q8, qs = O.quant_pertoken(q)
    k8, ks = O.quant_pertoken(k)
    v8 = torch.full((1, 1, 16, 8), 100, dtype=torch.int8)
    vs = torch.tensor([[0.02]], dtype=torch.float16)
    sm = 0.35
    got = O.attention_full_int8(q8, k8, v8, qs, ks, vs, False, sm, block_m=16, block_n=16).float()
    x = (q8.float() @ k8.float().transpose(2, 3)) * qs.float()[..., None] * ks.float()[:, :, None, :] * (sm * O.LOG2E)
    p = torch.exp2(x - x.max(dim=-1, keepdim=True).values)
    ratio = O.p_requant_reference(p).sum(-1) / (127 * p.sum(-1))
    want = 100 * float(vs) * ratio
    assert (got - want[..., None]).abs().max() < 2e-3
    assert 0.9 < ratio.mean() < 1.1


def test_l_sums_unquantised_p():
    """Rows whose probabilities all fall below 1/254 quantise to P8 == 0: the numerator vanishes, l does not."""
    N = 512
    q8 = torch.zeros((1, 1, N, 8), dtype=torch.int8)          # all logits equal -> p = 1 for the first block ...
    q8[..., 0] = 1
    k8 = torch.zeros((1, 1, N, 8), dtype=torch.int8)
    k8[0, 0, 0, 0] = 127                                       # ... except key 0 dominates by a wide margin
    v8 = torch.full((1, 1, N, 8), 50, dtype=torch.int8)
    v8[0, 0, 0] = 0
    one = torch.ones((1, 1, N), dtype=torch.float16)
    vs = torch.ones((1, 1), dtype=torch.float16)
    got = O.attention_full_int8(q8, k8, v8, one, one, vs, False, 0.1, block_m=N, block_n=N).float()
    # logits: key0 = 12.7, others 0 -> p_others = exp(-12.7) ~ 3e-6 each, P8 = 0; key 0 has V = 0
    assert torch.all(got == 0)
    exact = O.attention_exact(q8.half(), k8.half(), v8.half(), False, 0.1).float()
    assert exact.abs().max() > 0                               # the unquantised path keeps a little mass


@pytest.mark.parametrize("variant", ["full", "half"])
def test_causal_equals_dense_masked_evaluation(variant):
    q, k, v, _ = O.make_inputs(1, 2, 64, 16, seed=7)
    q8, qs = O.quant_pertoken(q)
    k8, ks = O.quant_pertoken(k)
    v8, vs = O.quant_pertensor(v)
    sm = 0.25
    x = (q8.float() @ k8.float().transpose(2, 3)) * qs.float()[..., None] * ks.float()[:, :, None, :]
    if variant == "half":
        got = O.attention_int8(q8, k8, v, qs, ks, True, sm, block_m=32, block_n=16).float()
        want = _dense_attention(x * sm, v.float(), True)
        tol = 2e-3
    else:
        got = O.attention_full_int8(q8, k8, v8, qs, ks, vs, True, sm, block_m=32, block_n=16).float()
        want = _dense_attention(x * sm, v8.float() * vs.float()[..., None, None], True)
        tol = 3e-2                                             # P8 has 1/127 resolution
    assert (got - want).abs().max() < tol
    # row 0 attends to key 0 only
    first = v.float()[:, :, 0] if variant == "half" else v8.float()[:, :, 0] * vs.float()[..., None]
    assert (got[:, :, 0] - first).abs().max() < 1e-2
    # a causal run never looks at keys above the diagonal: perturbing them changes nothing
    k8b = k8.clone(); k8b[:, :, 40:] = 0
    vb = v.clone(); vb[:, :, 40:] = 0
    v8b = v8.clone(); v8b[:, :, 40:] = 0
    if variant == "half":
        again = O.attention_int8(q8, k8b, vb, qs, ks, True, sm, block_m=32, block_n=16).float()
    else:
        again = O.attention_full_int8(q8, k8b, v8b, qs, ks, vs, True, sm, block_m=32, block_n=16).float()
    assert torch.equal(again[:, :, :40], got[:, :, :40])


def test_block_n_dependence_is_bounded_but_real():
    """P is quantised against the running maximum, so block_n changes the result a little (not zero)."""
    q, k, v, _ = O.make_inputs(1, 2, 256, 64, seed=8)
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    a = O.attention_full_int8(q8, k8, v8, qs, ks, vs, False, 0.125, block_n=128).float()
    b = O.attention_full_int8(q8, k8, v8, qs, ks, vs, False, 0.125, block_n=64).float()
    d = (a - b).abs().max().item()
    assert 0 < d < 2e-2


@pytest.mark.parametrize("causal", [False, True])
def test_ragged_length_equals_dense_softmax(causal):
    """N that is no multiple of the blocks: the blocked evaluation (shorter last block, shorter last row tile) must still
    equal torch.softmax attention over exactly N keys."""
    g = torch.Generator().manual_seed(12)
    N, D = 200, 32
    q = torch.randn((1, 2, N, D), generator=g).half()
    k = torch.randn((1, 2, N, D), generator=g).half()
    v = torch.randn((1, 2, N, D), generator=g).half()
    for bn in (64, 128):
        got = O.attention_fp(q, k, v, causal, 0.2, block_n=bn).float()
        want = _dense_attention(torch.matmul(q.float(), k.float().transpose(2, 3)) * 0.2, v.float(), causal)
        assert (got - want).abs().max() < 2e-3
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    a = O.attention_full_int8(q8, k8, v8, qs, ks, vs, causal, 0.2, block_n=64).float()
    assert torch.isfinite(a).all() and (a - want).abs().max() < 6e-2     # quantisation error only


# ------------------------------------------------------------------------------------------ split-KV
def test_splitkv_combine_reproduces_dense_softmax():
    g = torch.Generator().manual_seed(9)
    x = torch.randn((1, 2, 8, 24), generator=g) * 3           # logits, natural-log domain
    v = torch.randn((1, 2, 24, 4), generator=g)
    want = torch.softmax(x, dim=-1) @ v
    parts, lses = [], []
    for lo, hi in ((0, 8), (8, 16), (16, 24), (24, 24)):       # the last split is empty
        if lo == hi:
            parts.append(torch.zeros((1, 2, 8, 4))); lses.append(torch.full((1, 2, 8), float("-inf")))
            continue
        xs = x[..., lo:hi]
        parts.append(torch.softmax(xs, dim=-1) @ v[:, :, lo:hi])
        lses.append(torch.logsumexp(xs, dim=-1) * O.LOG2E)
    got, lse = O.splitkv_combine(torch.stack(parts), torch.stack(lses))
    assert (got - want).abs().max() < 1e-5
    assert (lse - torch.logsumexp(x, dim=-1) * O.LOG2E).abs().max() < 1e-4


def test_causal_split_ranges_cover_each_tiles_visible_blocks_once():
    for n, bm, bn, ns in ((1024, 128, 128, 3), (1000, 128, 64, 4), (256, 128, 64, 5), (130, 128, 128, 2)):
        n_blocks = -(-n // bn)
        for r0, r1, ranges in O.splitkv_ranges_causal(n, bm, bn, ns):
            vis = min(-(-(r0 + bm) // bn), n_blocks)                 # blocks that hold a key <= the tile's last row
            covered = [b for b0, b1 in ranges for b in range(b0, b1)]
            assert covered == list(range(vis)) and len(ranges) == ns
            assert max(b1 - b0 for b0, b1 in ranges) == -(-vis // ns)
    assert O.splitkv_ranges_causal(512, 128, 128, 2) == [(0, 128, [(0, 1), (1, 1)]), (128, 256, [(0, 1), (1, 2)]),
                                                         (256, 384, [(0, 2), (2, 3)]), (384, 512, [(0, 2), (2, 4)])]


def test_splitkv_ranges_follow_ceil_partition():
    assert O.splitkv_ranges(1024, 128, 3) == [(0, 3), (3, 6), (6, 8)]
    assert O.splitkv_ranges(256, 128, 4) == [(0, 1), (1, 2), (2, 2), (3, 2)]
    assert O.splitkv_ranges(512, 128, 1) == [(0, 4)]


@pytest.mark.parametrize("causal", [False, True])
def test_full_int8_split_agrees_with_single_pass(causal):
    q, k, v, _ = O.make_inputs(1, 2, 256, 32, seed=10)
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    one = O.attention_full_int8(q8, k8, v8, qs, ks, vs, causal, 0.2, block_m=64, block_n=64).float()
    same = O.attention_full_int8_splitkv(q8, k8, v8, qs, ks, vs, causal, 0.2, 1, block_m=64, block_n=64).float()
    assert (one - same).abs().max() < 1e-3                     # one split: identical up to the fp16 store
    two = O.attention_full_int8_splitkv(q8, k8, v8, qs, ks, vs, causal, 0.2, 2, block_m=64, block_n=64).float()
    assert (one - two).abs().max() < 2e-2                      # later splits quantise P against their own maximum


def test_exact_attention_matches_reference_recipe():
    q, k, v, _ = O.make_inputs(1, 1, 16, 8, seed=11, std=0.5)
    got = O.attention_exact(q, k, v, True, 1.0).float()
    want = _dense_attention(q.float() @ k.float().transpose(2, 3), v.float(), True)
    assert (got - want).abs().max() < 2e-3


# ---- per-block, per-channel V scales (layout of the reference's CUDA kernel, csrc/flash_fwd_kernel_full_qi8.h:156-160)
def test_quant_perblock_channel_against_python_loop_and_invariants():
    g = torch.Generator().manual_seed(12)
    x = (torch.randn((1, 2, 20, 4), generator=g) * 2).half()
    x[0, 1, 8:16, 2] = 0                                       # an all-zero (block, channel)
    q, s = O.quant_perblock_channel(x, 8)
    assert q.dtype == torch.int8 and q.shape == x.shape and s.shape == (1, 2, 3, 4) and s.dtype == torch.float32
    for h in range(2):
        for blk in range(3):
            rows = range(8 * blk, min(8 * blk + 8, 20))
            for c in range(4):
                col = [np.float32(float(x[0, h, r, c])) for r in rows]
                amax = max(abs(t) for t in col)
                sc = np.float32(amax) / np.float32(127)
                assert float(s[0, h, blk, c]) == float(sc)
                for r, t in zip(rows, col):
                    want = 0 if sc == 0 else int(np.rint(np.float32(t) / sc))
                    assert int(q[0, h, r, c]) == want
                if amax > 0:
                    assert max(abs(int(q[0, h, r, c])) for r in rows) == 127
    assert int(q[0, 1, 8:16, 2].abs().max()) == 0 and float(s[0, 1, 1, 2]) == 0.0


@pytest.mark.parametrize("causal", [False, True])
def test_blocked_v_scale_filled_with_the_scalar_is_the_scalar_form(causal):
    q, k, v, _ = O.make_inputs(1, 2, 192, 32, seed=13)
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    want = O.attention_full_int8(q8, k8, v8, qs, ks, vs, causal, 0.2, block_m=64, block_n=64)
    vs4 = vs.float()[:, :, None, None].expand(1, 2, 3, 32).contiguous()
    got = O.attention_full_int8(q8, k8, v8, qs, ks, vs4, causal, 0.2, block_m=64, block_n=64, v_scale_block=64)
    assert torch.equal(got, want)
    vs4b = vs.float()[:, :, None, None].expand(1, 2, 2, 32).contiguous()         # one scale row per two key blocks
    got = O.attention_full_int8(q8, k8, v8, qs, ks, vs4b, causal, 0.2, block_m=64, block_n=64, v_scale_block=128)
    assert torch.equal(got, want)


def test_blocked_v_scale_equals_scalar_form_on_prescaled_v():
    # power-of-two factors per (block, channel) commute exactly with the integer products: scaling V8 by 2^e and
    # using the scalar form gives the same fp32 numbers as the factors applied to the accumulator, as long as the
    # scaled V stays exactly representable (done here in the integer domain with small V)
    g = torch.Generator().manual_seed(14)
    q, k, _, _ = O.make_inputs(1, 1, 128, 16, seed=14)
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k)
    v8 = torch.randint(-15, 16, (1, 1, 128, 16), generator=g, dtype=torch.int8)
    e = torch.randint(0, 4, (1, 1, 2, 16), generator=g)
    fac = torch.pow(2.0, e.float())                                              # [1,1,2,16], block of 64 keys
    v8_scaled = (v8.view(1, 1, 2, 64, 16).float() * fac[:, :, :, None, :]).view(1, 1, 128, 16).to(torch.int8)
    assert int(v8_scaled.abs().max()) <= 127
    one = torch.ones((1, 1))
    want = O.attention_full_int8(q8, k8, v8_scaled, qs, ks, one, False, 0.3, block_m=64, block_n=64, out_dtype=torch.float32)
    got = O.attention_full_int8(q8, k8, v8, qs, ks, fac, False, 0.3, block_m=64, block_n=64, v_scale_block=64,
                                out_dtype=torch.float32)
    assert torch.equal(got, want)


def test_v_scale_rows_shorter_than_the_key_block():
    """64-key scale rows under a 128-key softmax block (the reference kernel's kBlockN = 64 granularity of V scales)."""
    g = torch.Generator().manual_seed(24)
    q, k, _, _ = O.make_inputs(1, 2, 256, 16, seed=24)
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k)
    v8 = torch.randint(-15, 16, (1, 2, 256, 16), generator=g, dtype=torch.int8)
    # (a) power-of-two factors per (64-key row, channel) equal the scalar form on V pre-multiplied by them, up to the
    # order of two fp32 additions
    e = torch.randint(0, 4, (1, 2, 4, 16), generator=g)
    fac = torch.pow(2.0, e.float())
    v8_scaled = (v8.view(1, 2, 4, 64, 16).float() * fac[:, :, :, None, :]).view(1, 2, 256, 16).to(torch.int8)
    one = torch.ones((1, 2))
    for causal in (False, True):
        want = O.attention_full_int8(q8, k8, v8_scaled, qs, ks, one, causal, 0.3, block_n=128, out_dtype=torch.float32)
        got = O.attention_full_int8(q8, k8, v8, qs, ks, fac, causal, 0.3, block_n=128, v_scale_block=64, out_dtype=torch.float32)
        assert torch.allclose(got, want, rtol=2e-6, atol=1e-6)
        assert not torch.allclose(got, O.attention_full_int8(q8, k8, v8, qs, ks, fac.flip(2), causal, 0.3, block_n=128,
                                                             v_scale_block=64, out_dtype=torch.float32), rtol=1e-3)
    # (b) one key block: the result is attention with the weights P8 / 127 over V dequantised row by row, divided by the
    # sum of the unquantised p - evaluated densely in float64 from the definition
    q8b, k8b, v8b, qsb, ksb = q8[:, :, :128], k8[:, :, :128], v8[:, :, :128], qs[:, :, :128], ks[:, :, :128]
    rows = torch.rand((1, 2, 2, 16), generator=g) + 0.5
    got = O.attention_full_int8(q8b, k8b, v8b, qsb, ksb, rows, False, 0.3, block_n=128, v_scale_block=64, out_dtype=torch.float32)
    x = O.qk_int32(q8b, k8b).float() * qsb.float()[..., None] * ksb.float()[:, :, None, :]
    c = float(torch.tensor(0.3, dtype=torch.float32) * torch.tensor(O.LOG2E, dtype=torch.float32))
    m = x.max(dim=-1).values * c
    p = torch.exp2(x * c - m[..., None])
    p8 = O.p_requant_reference(p).double()
    vf = v8b.double() * rows.double().repeat_interleave(64, dim=2)             # key r uses scale row r // 64
    want = (p8 / 127) @ vf / p.double().sum(dim=-1, keepdim=True)
    assert (got.double() - want).abs().max().item() < 1e-5 * want.abs().max().item()


def test_blocked_v_scale_is_more_accurate_with_an_outlier_channel_burst():
    q, k, v, _ = O.make_inputs(1, 2, 256, 32, seed=15)
    v = v.clone(); v[:, :, 64:128, 5] *= 30                                     # a burst in one channel of one key block
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k)
    exact = O.attention_exact(q, k, v, False, 0.2).float()
    v8s, vss = O.quant_pertensor(v)
    coarse = O.attention_full_int8(q8, k8, v8s, qs, ks, vss, False, 0.2, block_m=64, block_n=64).float()
    v8b, vsb = O.quant_perblock_channel(v, 64)
    fine = O.attention_full_int8(q8, k8, v8b, qs, ks, vsb, False, 0.2, block_m=64, block_n=64, v_scale_block=64).float()
    other = [c for c in range(32) if c != 5]
    err_c = (coarse - exact)[..., other].abs().mean()
    err_f = (fine - exact)[..., other].abs().mean()
    assert err_f < 0.5 * err_c                                                   # the burst no longer sets every channel's step


def test_blocked_v_scale_split_agrees_with_single_pass():
    q, k, v, _ = O.make_inputs(1, 2, 256, 32, seed=16)
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_perblock_channel(v, 64)
    one = O.attention_full_int8(q8, k8, v8, qs, ks, vs, False, 0.2, block_m=64, block_n=64, v_scale_block=64).float()
    two = O.attention_full_int8_splitkv(q8, k8, v8, qs, ks, vs, False, 0.2, 2, block_m=64, block_n=64, v_scale_block=64).float()
    # (the second split quantises P against its own maximum: same size of deviation as with a scalar V scale)
    assert (one - two).abs().max() < 3e-2 and (one - two).abs().mean() < 2e-3


def test_separate_query_and_key_lengths_are_row_slices_of_the_square_case():
    q, k, v, _ = O.make_inputs(1, 2, 200, 32, seed=17)
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    square = O.attention_full_int8(q8, k8, v8, qs, ks, vs, False, 0.2, block_m=64, block_n=64)
    part = O.attention_full_int8(q8[:, :, 70:75], k8, v8, qs[:, :, 70:75], ks, vs, False, 0.2, block_m=64, block_n=64)
    assert part.shape == (1, 2, 5, 32) and torch.equal(part, square[:, :, 70:75])
    half = O.attention_int8(q8[:, :, :3], k8, v, qs[:, :, :3], ks, False, 0.2, block_m=64, block_n=64)
    assert torch.equal(half, O.attention_int8(q8, k8, v, qs, ks, False, 0.2, block_m=64, block_n=64)[:, :, :3])
    two = O.attention_full_int8_splitkv(q8[:, :, 70:75], k8, v8, qs[:, :, 70:75], ks, vs, False, 0.2, 2, block_m=64, block_n=64)
    assert torch.equal(two, O.attention_full_int8_splitkv(q8, k8, v8, qs, ks, vs, False, 0.2, 2, block_m=64, block_n=64)[:, :, 70:75])


@pytest.mark.parametrize("variant", ["full", "half", "fp"])
@pytest.mark.parametrize("nq", [1, 37, 64, 130])
def test_causal_with_more_keys_than_queries_is_the_tail_of_the_square_problem(variant, nq):
    """Bottom-right aligned mask (csrc/mask.h:53,172): the last nq query rows against all N keys must equal the last nq
    rows of the square causal evaluation, bit for bit."""
    N = 200
    q, k, v, _ = O.make_inputs(1, 2, N, 32, seed=18)
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    t = slice(N - nq, N)
    kw = dict(block_m=64, block_n=64)
    if variant == "full":
        sq = O.attention_full_int8(q8, k8, v8, qs, ks, vs, True, 0.2, **kw)
        part = O.attention_full_int8(q8[:, :, t], k8, v8, qs[:, :, t], ks, vs, True, 0.2, **kw)
    elif variant == "half":
        sq = O.attention_int8(q8, k8, v, qs, ks, True, 0.2, **kw)
        part = O.attention_int8(q8[:, :, t], k8, v, qs[:, :, t], ks, True, 0.2, **kw)
    else:
        sq = O.attention_fp(q, k, v, True, 0.2, **kw)
        part = O.attention_fp(q[:, :, t], k, v, True, 0.2, **kw)
    assert torch.equal(part, sq[:, :, t])


def test_causal_with_fewer_keys_than_queries_leaves_the_first_rows_empty():
    q, k, v, _ = O.make_inputs(1, 1, 100, 16, seed=19)
    nk = 30                                                                      # row i sees keys 0 .. i - 70
    o, lse = O.attention_fp(q, k[:, :, :nk], v[:, :, :nk], True, 0.3, block_m=64, block_n=64, return_lse=True)
    assert o[:, :, :70].abs().max().item() == 0 and torch.isinf(lse[:, :, :70]).all() and (lse[:, :, :70] < 0).all()
    p = (q.float() @ k[:, :, :nk].float().transpose(2, 3)) * 0.3
    keep = (torch.arange(100)[:, None] - 70) >= torch.arange(nk)[None, :]
    want = torch.softmax(p.masked_fill(~keep, float("-inf"))[:, :, 70:], dim=-1) @ v[:, :, :nk].float()
    assert (o[:, :, 70:].float() - want).abs().max().item() < 2e-3


# ------------------------------------------------------------------------------------------ appending to an int8 cache
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_kvcache_append_equals_quantising_the_concatenation(dtype):
    """K rows are quantised independently, so a cache filled by two appends must equal quant_pertoken of the concatenation
    bit for bit (values and scales); V with the concatenation's per-(batch, head) scale must equal quant_pertensor's rows.
    Entries are filled to different lengths; rows outside the appended ranges stay as they were."""
    torch.manual_seed(41)
    Z, H, d, n_cache = 2, 3, 32, 40
    first, second = 7, 5
    k = torch.randn((Z, H, first + second, d)).to(dtype); v = torch.randn((Z, H, first + second, d)).to(dtype)
    k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    kc = torch.full((Z, H, n_cache, d), 99, dtype=torch.int8); vc = torch.full((Z, H, n_cache, d), 99, dtype=torch.int8)
    ksc = torch.full((Z, H, n_cache), -1.0, dtype=dtype)
    start = [0, 11]
    O.kvcache_append(kc, ksc, k[:, :, :first], start, vc, vs, v[:, :, :first])
    O.kvcache_append(kc, ksc, k[:, :, first:], [s + first for s in start], vc, vs, v[:, :, first:])
    # (in bf16 the quotient of the largest element can round up to 128, which the harness's quantiser wraps to -128,
    # benchmark.py:106; the append saturates such elements instead: they are compared apart)
    over = torch.round(v / vs[:, :, None, None]).abs() > 127
    assert dtype == torch.bfloat16 or not over.any()
    for b in range(Z):
        r = slice(start[b], start[b] + first + second)
        assert torch.equal(kc[b, :, r], k8[b]) and torch.equal(ksc[b, :, r], ks[b])
        assert torch.equal(vc[b, :, r][~over[b]], v8[b][~over[b]]) and (vc[b, :, r][over[b]].abs() == 127).all()
        keep = torch.ones(n_cache, dtype=torch.bool); keep[r] = False
        assert (kc[b][:, keep] == 99).all() and (vc[b][:, keep] == 99).all() and (ksc[b][:, keep] == -1).all()


def test_kvcache_append_saturates_v_and_drops_rows_past_the_end():
    Z, H, d, n_cache = 1, 1, 16, 4
    kc = torch.zeros((Z, H, n_cache, d), dtype=torch.int8); vc = torch.zeros_like(kc)
    ksc = torch.zeros((Z, H, n_cache), dtype=torch.float16)
    k_new = torch.arange(3 * d, dtype=torch.float32).reshape(1, 1, 3, d).half() - 20
    v_new = torch.tensor([[-1000.0, -2.0, -0.26, 0.0, 0.24, 0.26, 1.0, 126.9, 127.4, 500.0] + [0.0] * 6] * 3).reshape(1, 1, 3, d).half()
    vs = torch.tensor([[1.0]], dtype=torch.float16)
    O.kvcache_append(kc, ksc, k_new, [2], vc, vs, v_new)                        # room for two of the three rows
    assert vc[0, 0, 2, :10].tolist() == [-127, -2, 0, 0, 0, 0, 1, 127, 127, 127]  # round-half-even, saturated
    assert torch.equal(vc[0, 0, 3], vc[0, 0, 2]) and (vc[0, 0, :2] == 0).all()
    want8, wants = O.quant_pertoken(k_new)
    assert torch.equal(kc[0, 0, 2:], want8[0, 0, :2]) and torch.equal(ksc[0, 0, 2:], wants[0, 0, :2]) and (kc[0, 0, :2] == 0).all()
    zs = torch.zeros((1, 1), dtype=torch.float16)
    O.kvcache_append(kc, ksc, k_new[:, :, :1], [0], vc, zs, torch.zeros((1, 1, 1, d)).half())   # 0 / 0 -> 0
    assert (vc[0, 0, 0] == 0).all()
