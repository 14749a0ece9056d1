"""GPU parity tests: the HIP kernels, called through the C ABI of libintfa.so, against the CPU oracle on
the same seeded inputs; plus size-independent properties at the full benchmark shapes.

Tolerances (stated by the task for this path): int32 QK^T accumulators bit-exact; fp16 output within
max-abs 2e-2 and mean-rel 1e-2 of the reference's quantised arithmetic, where
mean-rel = mean|a - b| / mean|b| over all elements.  Against the oracle evaluated with the kernel's own
P rounding the agreement is far tighter (only exp2 differs in the last place) and is asserted as such.
"""
import math

import pytest
import torch

import intfa_oracle as O
import int_flashattention_amd as M

pytestmark = pytest.mark.gpu
DEV = "cuda"
MAX_ABS, MEAN_REL = 2e-2, 1e-2


def mean_rel(a, b):
    a, b = a.float().cpu(), b.float().cpu()
    return ((a - b).abs().mean() / b.abs().mean()).item()


def max_abs(a, b):
    return (a.float().cpu() - b.float().cpu()).abs().max().item()


def quantised(B, H, N, D, seed, dtype=torch.float16, std=1.0, **kw):
    q, k, v, cols = O.make_inputs(B, H, N, D, seed=seed, dtype=dtype, std=std, **kw)
    q8, qs = O.quant_pertoken(q)
    k8, ks = O.quant_pertoken(k)
    v8, vs = O.quant_pertensor(v)
    return dict(q=q, k=k, v=v, q8=q8, k8=k8, v8=v8, qs=qs, ks=ks, vs=vs)


def gpu(*ts):
    return [t.to(DEV) for t in ts]


def run_full(x, causal, sm, **kw):
    o = M.attention_full_int8(*gpu(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"]), causal, sm, **kw)
    torch.cuda.synchronize()
    return o


# ------------------------------------------------------------------------------------------ int32 S
@pytest.mark.parametrize("D", [64, 128])
def test_qk_int32_accumulators_bit_exact(D):
    x = quantised(2, 3, 384, D, seed=5)
    s = M.debug_qk_int32(*gpu(x["q8"], x["k8"])).cpu()
    assert torch.equal(s, O.qk_int32(x["q8"], x["k8"]))


def test_qk_int32_extreme_values():
    q8 = torch.full((1, 1, 128, 128), 127, dtype=torch.int8)
    k8 = torch.full((1, 1, 128, 128), -127, dtype=torch.int8)
    k8[0, 0, ::2] = 127
    s = M.debug_qk_int32(*gpu(q8, k8)).cpu()
    assert torch.equal(s, O.qk_int32(q8, k8))
    assert s.abs().max().item() == 127 * 127 * 128


# ------------------------------------------------------------------------------------------ full-int8
@pytest.mark.parametrize("B,H,N,D,causal", [
    (1, 4, 256, 64, False),        # the benchmark's CPU-runnable configuration
    (1, 4, 256, 128, False),
    (1, 2, 512, 128, True),
    (2, 3, 384, 64, True),
    (1, 2, 1024, 128, False),
])
@pytest.mark.parametrize("p_round", ["rne", "reference"])
def test_full_int8_matches_oracle(B, H, N, D, causal, p_round):
    x = quantised(B, H, N, D, seed=11)
    sm = D ** -0.5
    o = run_full(x, causal, sm, p_round=p_round)
    assert o.dtype == torch.float16 and o.shape == (B, H, N, D) and o.is_contiguous()
    ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], causal, sm, block_n=128)
    assert max_abs(o, ref) <= MAX_ABS and mean_rel(o, ref) <= MEAN_REL
    same = ref if p_round == "reference" else O.attention_full_int8(
        x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], causal, sm, block_n=128, p_requant=O.p_requant_rne)
    assert max_abs(o, same) <= 4e-3 and mean_rel(o, same) <= 2e-4
    exact = O.attention_exact(x["q"], x["k"], x["v"], causal, sm)
    assert max_abs(o, exact) <= 6e-2                        # quantisation error itself, reported by the bench


@pytest.mark.parametrize("d", [16, 32])
def test_small_head_dims_are_accepted(d):
    x = quantised(1, 2, 256, d, seed=12)
    sm = d ** -0.5
    o = run_full(x, False, sm, p_round="reference")
    ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], False, sm, block_n=128)
    assert o.shape == (1, 2, 256, d)
    assert max_abs(o, ref) <= 4e-3


def test_bf16_inputs_and_output():
    """bf16 Q/K/V and bf16 scales, bf16 output (beyond the reference wrappers, which hard-code fp16 out)."""
    x = quantised(2, 2, 256, 64, seed=13, dtype=torch.bfloat16, std=0.5)
    assert x["qs"].dtype == torch.bfloat16
    o = run_full(x, False, 0.125, out_dtype=torch.bfloat16, p_round="reference")
    assert o.dtype == torch.bfloat16
    ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], False, 0.125,
                                block_n=128, out_dtype=torch.bfloat16)
    assert max_abs(o, ref) <= 8e-3 and mean_rel(o, ref) <= 5e-3   # bf16 keeps 8 bits of mantissa


def test_outlier_channels_stress_per_token_scales():
    x = quantised(1, 2, 512, 128, seed=14, k_outlier_frac=0.01, k_outlier_gain=20.0)
    sm = 128 ** -0.5
    o = run_full(x, True, sm, p_round="reference")
    ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], True, sm, block_n=128)
    assert max_abs(o, ref) <= 6e-3 and mean_rel(o, ref) <= 1e-3


def test_strided_inputs_equal_contiguous():
    x = quantised(2, 4, 256, 128, seed=15)
    sm = 0.1
    base = run_full(x, True, sm)
    # [B, N, H, d] storage viewed as [B, H, N, d]
    q8, k8, v8 = (t.permute(0, 2, 1, 3).contiguous().to(DEV).permute(0, 2, 1, 3) for t in (x["q8"], x["k8"], x["v8"]))
    qs, ks = (t.transpose(1, 2).contiguous().to(DEV).transpose(1, 2) for t in (x["qs"], x["ks"]))
    assert not q8.is_contiguous() and not qs.is_contiguous()
    o = M.attention_full_int8(q8, k8, v8, qs, ks, x["vs"].to(DEV), True, sm)
    assert torch.equal(o, base)


def test_lse_output():
    x = quantised(1, 2, 256, 64, seed=16)
    o, lse = M.attention_full_int8(*gpu(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"]), False, 0.125,
                                   p_round="reference", return_lse=True)
    _, ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], False, 0.125, return_lse=True)
    assert (lse.cpu() - ref).abs().max().item() < 1e-3


# ------------------------------------------------------------------------------------------ split-KV
@pytest.mark.parametrize("causal,splits", [(False, 2), (True, 3), (True, 8)])
def test_split_kv_matches_oracle_split(causal, splits):
    x = quantised(1, 2, 1024, 128, seed=17)
    sm = 128 ** -0.5
    o = run_full(x, causal, sm, num_splits=splits, p_round="reference")
    ref = O.attention_full_int8_splitkv(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], causal, sm, splits, block_n=128)
    assert max_abs(o, ref) <= 4e-3 and mean_rel(o, ref) <= 2e-4
    # A split restarts the running maximum, so its P is quantised against a different reference than in the
    # single pass: the two evaluations differ by the P8 quantisation noise (the oracle shows the same gap).
    single = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], causal, sm, block_n=128)
    assert max_abs(o, single) <= MAX_ABS and mean_rel(o, single) <= 2e-2
    assert abs(mean_rel(o, single) - mean_rel(ref, single)) <= 1e-3


# ------------------------------------------------------------------------------------------ full-size properties
def _headline_inputs(B=4, H=32, N=4096, D=128, seed=20):
    g = torch.Generator(device=DEV).manual_seed(seed)
    mk = lambda: torch.randn((B, H, N, D), generator=g, device=DEV, dtype=torch.float16)
    q8, qs = M.quant_pertoken(mk())
    k8, ks = M.quant_pertoken(mk())
    v8, vs = M.quant_pertensor(mk())
    return q8, k8, v8, qs, ks, vs


def test_headline_shape_slices_reproduce_and_v_scale_is_linear():
    B, H, N, D = 4, 32, 4096, 128
    q8, k8, v8, qs, ks, vs = _headline_inputs()
    sm = D ** -0.5
    o = M.attention_full_int8(q8, k8, v8, qs, ks, vs, False, sm)
    assert torch.isfinite(o).all()
    # every (batch, head) is independent: recomputing one slice alone gives the same bits
    for b, h in ((0, 0), (3, 31), (1, 17)):
        sl = lambda t: t[b:b + 1, h:h + 1].contiguous()
        o1 = M.attention_full_int8(sl(q8), sl(k8), sl(v8), sl(qs), sl(ks), sl(vs), False, sm)
        assert torch.equal(o1, o[b:b + 1, h:h + 1])
    # the value scale is applied once, linearly: doubling it doubles the output exactly (power of two)
    o2 = M.attention_full_int8(q8, k8, v8, qs, ks, vs * 2, False, sm)
    assert torch.equal(o2, o * 2)
    # one slice against the CPU oracle at full sequence length
    b, h = 2, 5
    cpu = lambda t: t[b:b + 1, h:h + 1].cpu()
    ref = O.attention_full_int8(cpu(q8), cpu(k8), cpu(v8), cpu(qs), cpu(ks), cpu(vs), False, sm, block_n=128,
                                p_requant=O.p_requant_rne)
    assert max_abs(o[b:b + 1, h:h + 1], ref) <= 2e-3 and mean_rel(o[b:b + 1, h:h + 1], ref) <= 2e-4


def test_constant_v_gives_constant_columns_at_full_size():
    B, H, N, D = 2, 8, 4096, 128
    q8, k8, _, qs, ks, _ = _headline_inputs(B, H, N, D, seed=21)
    v8 = torch.full((B, H, N, D), 64, dtype=torch.int8, device=DEV)
    vs = torch.full((B, H), 1 / 64, dtype=torch.float16, device=DEV)
    o = M.attention_full_int8(q8, k8, v8, qs, ks, vs, True, D ** -0.5)
    # O = sum(P8) / (127 l): the same for every column of a row, and close to one
    assert torch.equal(o, o[..., :1].expand_as(o))
    assert (o.float() - 1).abs().max().item() < 0.05
    assert torch.equal(o[:, :, 0], torch.ones_like(o[:, :, 0]))    # row 0 sees key 0 only: P8 = 127, l = 1
