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


def assert_same_rounding(o, same):
    """Kernel against the oracle evaluated with the kernel's own P rounding.  The two differ only through exp2 in the
    last place, which now and then moves a value of 127 p across a rounding boundary: that one P8 step shows up in a
    single row as (v8 * v_scale / 127 l) of one key.  So: tight in the mean, tight in nearly every row, and no row
    beyond the overall bound."""
    d = (o.float().cpu() - same.float().cpu()).abs()
    rows = d.amax(dim=-1)
    assert mean_rel(o, same) <= 2e-4
    assert d.max().item() <= MAX_ABS
    assert (rows > 4e-3).float().mean().item() <= 2e-3


def quantised(B, H, N, D, seed, dtype=torch.float16, std=1.0, **kw):
    q, k, v, cols = O.make_inputs(B, H, N, D, seed=seed, dtype=dtype, std=std, **kw)
    q8, qs = O.quant_pertoken(q)
    k8, ks = O.quant_pertoken(k)
    v8, vs = O.quant_pertensor(v)
    return dict(q=q, k=k, v=v, q8=q8, k8=k8, v8=v8, qs=qs, ks=ks, vs=vs)


def gpu(*ts):
    return [t.to(DEV) for t in ts]


def run_full(x, causal, sm, **kw):
    kw.setdefault("p_round", "rne")      # (the tests that mean the entry point's default rounding call it directly)
    o = M.attention_full_int8(*gpu(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"]), causal, sm, **kw)
    torch.cuda.synchronize()
    return o


# ------------------------------------------------------------------------------------------ int32 S
@pytest.mark.parametrize("D", [64, 128, 256])
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
    (1, 2, 256, 256, False),       # head_dim 256 runs with 64-key blocks
    (2, 2, 384, 256, True),
    (1, 2, 512, 256, True),        # four query blocks: two per workgroup
])
@pytest.mark.parametrize("p_round", ["rne", "reference"])
def test_full_int8_matches_oracle(B, H, N, D, causal, p_round):
    x = quantised(B, H, N, D, seed=11)
    sm = D ** -0.5
    bn = M.block_n("full", D)
    assert bn == (128 if D == 128 else 64)
    o, lse = run_full(x, causal, sm, p_round=p_round, return_lse=True)
    assert o.dtype == torch.float16 and o.shape == (B, H, N, D) and o.is_contiguous()
    ref, lse_ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], causal, sm, block_n=bn,
                                         return_lse=True)
    assert max_abs(o, ref) <= MAX_ABS and mean_rel(o, ref) <= MEAN_REL
    assert (lse.cpu() - lse_ref).abs().max().item() <= 1e-3         # every row's LSE in its own slot
    same = ref if p_round == "reference" else O.attention_full_int8(
        x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], causal, sm, block_n=bn, p_requant=O.p_requant_rne)
    assert_same_rounding(o, same)
    exact = O.attention_exact(x["q"], x["k"], x["v"], causal, sm)
    assert max_abs(o, exact) <= 6e-2                        # quantisation error itself, reported by the bench


@pytest.mark.parametrize("D", [64, 128, 256])
def test_rne_rounding_against_reference_rounding_on_short_causal_rows(D):
    """The opt-in rounding of P ("rne": 127 p evaluated in fp32, rounded to nearest even) against the reference's fp16
    sequence (flash_atten_full_int8.py:49-51).  The two agree except where 127 p lies within an fp16 rounding of a .5
    boundary, and then by one step of 1/127.  On a row with many keys a step is invisible; on the first rows of a
    causal problem (row i sees i + 1 keys) one step moves the output by up to |v| / (127 l), l >= 1: with |v| up to the
    value range's maximum (about 4.5 for N(0,1) inputs) that is 3.5e-2, above the 2e-2 that holds everywhere else.
    Pinned here: rows with more than 16 keys stay inside 2e-2, the short rows inside two such steps, the mean inside 1e-2;
    the entry point's default is p_round="reference" (bit-for-bit the oracle's P8)."""
    B, H, N = 4, 8, 256
    x = quantised(B, H, N, D, seed=61 + D)
    sm = D ** -0.5
    bn = M.block_n("full", D)
    o = run_full(x, True, sm, p_round="rne")
    ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], True, sm, block_n=bn)
    d = (o.float().cpu() - ref.float()).abs()
    vmax = x["v"].float().abs().amax().item()
    step = vmax / 127
    assert mean_rel(o, ref) <= MEAN_REL
    assert d[:, :, 16:].max().item() <= MAX_ABS
    assert d[:, :, :16].max().item() <= 2 * step
    # and the reference rounding itself reproduces the oracle to the accuracy of exp2
    assert_same_rounding(run_full(x, True, sm, p_round="reference"), ref)


@pytest.mark.parametrize("D", [64, 128, 256])
def test_positional_call_uses_the_reference_rounding(D):
    """The drop-in call - positional arguments only, as the reference's callers write it - requantises P with the reference's
    own fp16 sequence (flash_atten_full_int8.py:49-51): bit-equal to p_round="reference", and different from the opt-in
    "rne" somewhere on a problem of this size."""
    x = quantised(2, 2, 384, D, seed=75 + D)
    sm = D ** -0.5
    args = gpu(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"])
    o = M.attention_full_int8(*args, False, sm)
    assert torch.equal(o, M.attention_full_int8(*args, False, sm, p_round="reference"))
    assert not torch.equal(o, M.attention_full_int8(*args, False, sm, p_round="rne"))
    ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], False, sm, block_n=M.block_n("full", D))
    assert_same_rounding(o, ref)


@pytest.mark.parametrize("d", [16, 32])
def test_small_head_dims_are_accepted(d):
    x = quantised(1, 2, 256, d, seed=12)
    sm = d ** -0.5
    o = run_full(x, False, sm, p_round="reference")
    assert M.block_n("full", d) == 64               # head dims 16 and 32 run the head_dim 64 kernel on zero-padded rows
    ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], False, sm, block_n=64)
    assert o.shape == (1, 2, 256, d)
    assert max_abs(o, ref) <= 4e-3


@pytest.mark.parametrize("d", [16, 32])
@pytest.mark.parametrize("causal", [False, True])
def test_small_head_dims_against_the_reference_admissible_key_block(d, causal):
    """The reference admits no key block longer than head_dim (tl.static_assert(BLOCK_N <= HEAD_DIM),
    flash_atten_full_int8.py:88), so at head_dim 16 / 32 its own runs requantise P per 16 / 32 keys at most.  This build
    evaluates those head dims with the 64-key block of the head_dim 64 kernel: another (coarser) frame for the running
    maximum, hence other P8.  The distance between the two frames is bounded here with the stated tolerance of this path:
    max-abs 2e-2, mean-rel 1e-2 against the oracle at block_n = head_dim, reference rounding on both sides."""
    x = quantised(2, 4, 512, d, seed=90 + d)
    sm = d ** -0.5
    o = run_full(x, causal, sm, p_round="reference")
    ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], causal, sm, block_n=d)
    print(f"d {d} causal {causal}: 64-key kernel vs oracle at block_n={d}: max-abs {max_abs(o, ref):.3e} mean-rel {mean_rel(o, ref):.3e}")
    assert max_abs(o, ref) <= MAX_ABS and mean_rel(o, ref) <= MEAN_REL


@pytest.mark.parametrize("bn_ref", [32, 16])
def test_head_dim_64_against_shorter_reference_key_blocks(bn_ref):
    """At head_dim 64 the reference's autotuner may also pick BLOCK_N = 32 or 16 (configs.py:13-19); its result depends on
    that choice (P8 is relative to the running maximum of the blocks seen so far).  The kernel's 64-key frame against those
    frames, with the stated tolerance: benchmark configuration 0 (B1 H4 N256 d64, N(0,1) inputs)."""
    x = quantised(1, 4, 256, 64, seed=20)
    sm = 64 ** -0.5
    o = run_full(x, False, sm, p_round="reference")
    ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], False, sm, block_n=bn_ref)
    print(f"config 0: 64-key kernel vs oracle at block_n={bn_ref}: max-abs {max_abs(o, ref):.3e} mean-rel {mean_rel(o, ref):.3e}")
    assert max_abs(o, ref) <= MAX_ABS and mean_rel(o, ref) <= MEAN_REL


def test_bf16_inputs_and_output():
    """bf16 Q/K/V and bf16 scales, bf16 output (beyond the reference wrappers, which hard-code fp16 out)."""
    x = quantised(2, 2, 256, 64, seed=13, dtype=torch.bfloat16, std=0.5)
    assert x["qs"].dtype == torch.bfloat16
    o = run_full(x, False, 0.125, out_dtype=torch.bfloat16, p_round="reference")
    assert o.dtype == torch.bfloat16
    ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], False, 0.125,
                                block_n=64, out_dtype=torch.bfloat16)
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
    base = run_full(x, True, sm, p_round="rne")
    # [B, N, H, d] storage viewed as [B, H, N, d]
    q8, k8, v8 = (t.permute(0, 2, 1, 3).contiguous().to(DEV).permute(0, 2, 1, 3) for t in (x["q8"], x["k8"], x["v8"]))
    qs, ks = (t.transpose(1, 2).contiguous().to(DEV).transpose(1, 2) for t in (x["qs"], x["ks"]))
    assert not q8.is_contiguous() and not qs.is_contiguous()
    o = M.attention_full_int8(q8, k8, v8, qs, ks, x["vs"].to(DEV), True, sm, p_round="rne")
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


@pytest.mark.parametrize("n,causal,splits,p_round", [(512, False, 2, "reference"), (512, True, 3, "reference"),
                                                    (512, False, 4, "rne"), (700, False, 3, "rne"), (640, True, 2, "rne")])
def test_split_kv_head_dim_256(n, causal, splits, p_round):
    """The head_dim 256 kernel (two waves per 32 query rows) against the oracle evaluated over the same key ranges, for
    both roundings of P: with the partition matched, only fp32 summation order and the output rounding are left."""
    x = quantised(1, 2, n, 256, seed=18)
    sm = 256 ** -0.5
    o = run_full(x, causal, sm, num_splits=splits, p_round=p_round)
    rq = O.p_requant_rne if p_round == "rne" else O.p_requant_reference
    ref = O.attention_full_int8_splitkv(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], causal, sm, splits, block_n=64,
                                        p_requant=rq)
    assert max_abs(o, ref) <= 4e-3 and mean_rel(o, ref) <= 2e-4


# ------------------------------------------------------------------------------------------ half-int8 and fp16
# No P requantisation on these paths: the only differences from the oracle are fp32 summation order inside the
# MFMA, the hardware exp2 and where the output is rounded to 16 bits, so the bounds are a few output ulps.
HALF_FP_CASES = [
    (1, 4, 256, 64, False, torch.float16),
    (1, 2, 512, 128, True, torch.float16),
    (2, 3, 384, 64, True, torch.float16),
    (1, 2, 256, 256, False, torch.float16),
    (1, 2, 384, 256, True, torch.float16),
    (2, 3, 300, 256, False, torch.bfloat16),     # ragged length, column halves
    (1, 2, 641, 256, True, torch.float16),
    (1, 2, 512, 128, True, torch.bfloat16),
    (2, 2, 256, 64, False, torch.bfloat16),
]


def _ulp_bounds(dtype):
    return (2e-3, 2e-4) if dtype == torch.float16 else (1.6e-2, 1.5e-3)


@pytest.mark.parametrize("B,H,N,D,causal,dtype", HALF_FP_CASES)
def test_half_int8_matches_oracle(B, H, N, D, causal, dtype):
    x = quantised(B, H, N, D, seed=31, dtype=dtype)
    sm = D ** -0.5
    bn = M.block_n("half", D)
    o, lse = M.attention_int8(*gpu(x["q8"], x["k8"], x["v"], x["qs"], x["ks"]), causal, sm, return_lse=True)
    torch.cuda.synchronize()
    assert o.dtype == dtype and o.shape == (B, H, N, D)
    ref, lse_ref = O.attention_int8(x["q8"], x["k8"], x["v"], x["qs"], x["ks"], causal, sm, block_n=bn, out_dtype=dtype,
                                    return_lse=True)
    ma, mr = _ulp_bounds(dtype)
    assert max_abs(o, ref) <= ma and mean_rel(o, ref) <= mr
    assert (lse.cpu() - lse_ref).abs().max().item() <= 2e-3
    if dtype == torch.float16:
        exact = O.attention_exact(x["q"], x["k"], x["v"], causal, sm)
        assert max_abs(o, exact) <= 4e-2 and mean_rel(o, exact) <= 2e-2     # int8 Q/K quantisation error itself


@pytest.mark.parametrize("B,H,N,D,causal,dtype", HALF_FP_CASES)
def test_fp16_attention_matches_oracle(B, H, N, D, causal, dtype):
    q, k, v, _ = O.make_inputs(B, H, N, D, seed=32, dtype=dtype)
    sm = D ** -0.5
    bn = M.block_n("fp", D)
    o, lse = M.attention(*gpu(q, k, v), causal, sm, return_lse=True)
    torch.cuda.synchronize()
    assert o.dtype == dtype and o.shape == (B, H, N, D)
    ref, lse_ref = O.attention_fp(q, k, v, causal, sm, block_n=bn, return_lse=True)
    ma, mr = _ulp_bounds(dtype)
    assert max_abs(o, ref) <= ma and mean_rel(o, ref) <= mr
    assert (lse.cpu() - lse_ref).abs().max().item() <= 2e-3
    exact = O.attention_exact(q, k, v, causal, sm)
    assert max_abs(o, exact) <= (2e-3 if dtype == torch.float16 else 1.6e-2)


@pytest.mark.parametrize("d", [16, 32])
def test_half_and_fp_small_head_dims(d):
    x = quantised(1, 2, 256, d, seed=33)
    sm = d ** -0.5
    o = M.attention_int8(*gpu(x["q8"], x["k8"], x["v"], x["qs"], x["ks"]), True, sm)
    ref = O.attention_int8(x["q8"], x["k8"], x["v"], x["qs"], x["ks"], True, sm, block_n=64)
    assert o.shape == (1, 2, 256, d) and max_abs(o, ref) <= 2e-3
    o = M.attention(*gpu(x["q"], x["k"], x["v"]), True, sm)
    ref = O.attention_fp(x["q"], x["k"], x["v"], True, sm, block_n=64)
    assert o.shape == (1, 2, 256, d) and max_abs(o, ref) <= 2e-3


@pytest.mark.parametrize("variant", ["half", "fp"])
@pytest.mark.parametrize("causal,splits,D", [(False, 2, 128), (True, 5, 64), (True, 3, 256)])
def test_half_and_fp_split_kv_equals_single_pass(variant, causal, splits, D):
    """Without P requantisation the split evaluation is the same sum in another order, except that P is cast to 16 bits
    relative to another running maximum (an independent 2^-11 relative rounding per element): it must agree with the
    single pass to a fraction of an output ulp in the mean, and its LSE to fp32 rounding."""
    x = quantised(1, 2, 1024, D, seed=34)
    sm = D ** -0.5
    if variant == "half":
        args = gpu(x["q8"], x["k8"], x["v"], x["qs"], x["ks"])
        f = M.attention_int8
    else:
        args = gpu(x["q"], x["k"], x["v"])
        f = M.attention
    o1, l1 = f(*args, causal, sm, return_lse=True)
    o2, l2 = f(*args, causal, sm, num_splits=splits, return_lse=True)
    torch.cuda.synchronize()
    assert max_abs(o2, o1) <= 1e-3 and mean_rel(o2, o1) <= 5e-4
    assert (l1 - l2).abs().max().item() <= 1e-3


@pytest.mark.parametrize("variant,N,D,splits", [("fp", 128, 64, 5), ("half", 384, 128, 2), ("full", 256, 256, 4), ("fp", 511, 256, 3)])
def test_causal_split_that_starts_inside_the_diagonal(variant, N, D, splits):
    """A split whose key range begins inside a query block's diagonal region holds no key at all for that block's first
    rows (their waves skip every block of the range): those rows must contribute nothing, not NaN."""
    x = quantised(2, 2, N, D, seed=37)
    sm = D ** -0.5
    if variant == "fp":
        o = M.attention(*gpu(x["q"], x["k"], x["v"]), True, sm, num_splits=splits)
        ref = O.attention_fp(x["q"], x["k"], x["v"], True, sm, block_n=64)
    elif variant == "half":
        o = M.attention_int8(*gpu(x["q8"], x["k8"], x["v"], x["qs"], x["ks"]), True, sm, num_splits=splits)
        ref = O.attention_int8(x["q8"], x["k8"], x["v"], x["qs"], x["ks"], True, sm, block_n=64)
    else:
        o = run_full(x, True, sm, num_splits=splits, p_round="reference")
        ref = O.attention_full_int8_splitkv(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], True, sm, splits,
                                            block_n=M.block_n("full", D))
    assert torch.isfinite(o).all()
    assert max_abs(o, ref) <= 4e-3 and mean_rel(o, ref) <= 3e-4


def test_half_int8_lse_matches_oracle():
    x = quantised(1, 2, 256, 128, seed=35)
    _, lse = M.attention_int8(*gpu(x["q8"], x["k8"], x["v"], x["qs"], x["ks"]), True, 0.09, return_lse=True)
    _, ref = O.attention_int8(x["q8"], x["k8"], x["v"], x["qs"], x["ks"], True, 0.09, block_n=64, return_lse=True)
    assert (lse.cpu() - ref).abs().max().item() < 1e-3


def test_three_variants_order_by_precision():
    """The reference's own evaluation (benchmark/benchmark_int.py: MRE of each variant against fp16 attention): the
    error against exact attention grows fp16 < half-int8 < full-int8, and every variant stays within a few percent."""
    x = quantised(1, 4, 1024, 128, seed=36)
    sm = 128 ** -0.5
    exact = O.attention_exact(x["q"], x["k"], x["v"], False, sm)
    e_fp = mean_rel(M.attention(*gpu(x["q"], x["k"], x["v"]), False, sm), exact)
    e_half = mean_rel(M.attention_int8(*gpu(x["q8"], x["k8"], x["v"], x["qs"], x["ks"]), False, sm), exact)
    e_full = mean_rel(run_full(x, False, sm, p_round="rne"), exact)
    assert e_fp < e_half < e_full < 5e-2


# ------------------------------------------------------------------------------------------ ragged sequence lengths
RAGGED = [(1, 2, 200, 128, False), (1, 2, 200, 128, True), (2, 3, 333, 64, False), (2, 3, 333, 64, True),
          (1, 2, 97, 128, True), (1, 2, 1, 64, False), (1, 2, 130, 256, False), (1, 2, 190, 256, True), (1, 4, 640 + 31, 128, False)]


@pytest.mark.parametrize("B,H,N,D,causal", RAGGED)
def test_ragged_lengths_full_int8(B, H, N, D, causal):
    """N that is not a multiple of 128 (nor of the key block): beyond the reference's Triton API, as in its CUDA tree."""
    x = quantised(B, H, N, D, seed=60)
    sm = D ** -0.5
    bn = M.block_n("full", D)
    s = M.debug_qk_int32(*gpu(x["q8"], x["k8"])).cpu()
    assert torch.equal(s, O.qk_int32(x["q8"], x["k8"]))
    o, lse = M.attention_full_int8(*gpu(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"]), causal, sm, return_lse=True, p_round="rne")
    torch.cuda.synchronize()
    assert o.shape == (B, H, N, D) and torch.isfinite(o).all()
    ref, lse_ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], causal, sm, block_n=bn,
                                         p_requant=O.p_requant_rne, return_lse=True)
    assert_same_rounding(o, ref)
    assert (lse.cpu() - lse_ref).abs().max().item() < 1e-3


@pytest.mark.parametrize("B,H,N,D,causal", RAGGED)
def test_ragged_lengths_half_and_fp(B, H, N, D, causal):
    x = quantised(B, H, N, D, seed=61)
    sm = D ** -0.5
    o = M.attention_int8(*gpu(x["q8"], x["k8"], x["v"], x["qs"], x["ks"]), causal, sm)
    ref = O.attention_int8(x["q8"], x["k8"], x["v"], x["qs"], x["ks"], causal, sm, block_n=64)
    assert o.shape == (B, H, N, D) and max_abs(o, ref) <= 2e-3 and mean_rel(o, ref) <= 3e-4
    o = M.attention(*gpu(x["q"], x["k"], x["v"]), causal, sm)
    ref = O.attention_fp(x["q"], x["k"], x["v"], causal, sm, block_n=64)
    assert max_abs(o, ref) <= 2e-3 and mean_rel(o, ref) <= 3e-4


@pytest.mark.parametrize("causal,splits", [(False, 3), (True, 2)])
def test_ragged_lengths_split_kv(causal, splits):
    x = quantised(1, 2, 700, 128, seed=62)
    sm = 128 ** -0.5
    o = run_full(x, causal, sm, num_splits=splits, p_round="reference")
    ref = O.attention_full_int8_splitkv(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], causal, sm, splits, block_n=128)
    assert max_abs(o, ref) <= 4e-3 and mean_rel(o, ref) <= 3e-4
    o1 = M.attention_int8(*gpu(x["q8"], x["k8"], x["v"], x["qs"], x["ks"]), causal, sm)
    o2 = M.attention_int8(*gpu(x["q8"], x["k8"], x["v"], x["qs"], x["ks"]), causal, sm, num_splits=splits)
    assert max_abs(o2, o1) <= 1e-3


def test_ragged_outputs_do_not_touch_memory_past_the_end():
    """Output rows are written for valid queries only: a guard region behind the output stays untouched."""
    x = quantised(1, 1, 130, 128, seed=63)
    o = run_full(x, False, 0.09, p_round="rne")
    ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], False, 0.09, p_requant=O.p_requant_rne)
    assert_same_rounding(o, ref)
    # the same call into a larger buffer through strides: rows 130.. of the buffer must keep their fill value
    import ctypes
    from int_flashattention_amd import _capi
    big = torch.full((1, 1, 256, 128), 7.0, dtype=torch.float16, device=DEV)
    q8, k8, v8, qs, ks, vs = gpu(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"])
    p = _capi.FwdParams()
    p.q, p.k, p.v, p.out = q8.data_ptr(), k8.data_ptr(), v8.data_ptr(), big.data_ptr()
    p.q_scale, p.k_scale, p.v_scale = qs.data_ptr(), ks.data_ptr(), vs.data_ptr()
    for name, t in (("q", q8), ("k", k8), ("v", v8), ("o", big)):
        setattr(p, f"{name}_stride_b", t.stride(0)); setattr(p, f"{name}_stride_h", t.stride(1)); setattr(p, f"{name}_stride_n", t.stride(2))
    p.qs_stride_b, p.qs_stride_h, p.qs_stride_n = qs.stride()
    p.ks_stride_b, p.ks_stride_h, p.ks_stride_n = ks.stride()
    p.vs_stride_b, p.vs_stride_h = vs.stride()
    p.batch, p.heads, p.seqlen, p.head_dim = 1, 1, 130, 128
    p.scale_dtype, p.io_dtype, p.causal, p.sm_scale, p.p_round, p.num_splits = 0, 0, 0, 0.09, _capi.PROUND_RNE, 1
    rc = _capi.load().intfa_fwd_full_int8(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert rc == 0
    assert torch.equal(big[:, :, :130], o) and (big[:, :, 130:] == 7.0).all()


# ------------------------------------------------------------------------------------------ separate key length
def _dense_cross(q, k, v, sm):
    s = torch.matmul(q.float(), k.float().transpose(2, 3)) * sm
    return torch.matmul(torch.softmax(s, dim=-1), v.float())


@pytest.mark.parametrize("B,H,Nq,Nk,D", [(2, 4, 1, 1000, 128), (1, 2, 128, 384, 64), (1, 3, 200, 77, 128), (1, 2, 130, 2048, 256)])
def test_separate_query_and_key_lengths(B, H, Nq, Nk, D):
    """Non-causal attention with Nq != Nk (decoding against a cache, cross attention): there is no oracle restatement
    with two lengths, so the check is the mathematics itself - int32 S against an integer matmul, outputs against dense
    softmax attention on the dequantised inputs within the quantisation error the equal-length cases show."""
    g = torch.Generator().manual_seed(70)
    q = torch.randn((B, H, Nq, D), generator=g).half()
    k = torch.randn((B, H, Nk, D), generator=g).half()
    v = torch.randn((B, H, Nk, D), generator=g).half()
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    sm = D ** -0.5
    s = M.debug_qk_int32(*gpu(q8, k8)).cpu()
    assert s.shape == (B, H, Nq, Nk) and torch.equal(s, O.qk_int32(q8, k8))
    exact = _dense_cross(q, k, v, sm)
    o = M.attention(*gpu(q, k, v), False, sm)
    assert o.shape == (B, H, Nq, D) and max_abs(o, exact) <= 2e-3
    qd, kd = q8.float() * qs.float()[..., None], k8.float() * ks.float()[..., None]
    o = M.attention_int8(*gpu(q8, k8, v, qs, ks), False, sm)
    assert max_abs(o, _dense_cross(qd, kd, v, sm)) <= 3e-3          # same dequantised Q, K: only fp16 P and output rounding
    vd = v8.float() * vs.float()[..., None, None]
    o = M.attention_full_int8(*gpu(q8, k8, v8, qs, ks, vs), False, sm, p_round="rne")
    assert max_abs(o, _dense_cross(qd, kd, vd, sm)) <= 3e-2 and mean_rel(o, _dense_cross(qd, kd, vd, sm)) <= 4e-2   # + P8 quantisation
    o2 = M.attention_full_int8(*gpu(q8, k8, v8, qs, ks, vs), False, sm, num_splits=3, p_round="rne")
    assert max_abs(o2, o) <= 2e-2


def test_decoding_shape_with_automatic_splits():
    """One query against a long cache: num_splits="auto" spreads the keys over many workgroups; the result equals the
    single pass (no P requantisation on the half-int8 path) and stays within the P8 noise on the full-int8 path."""
    g = torch.Generator().manual_seed(71)
    B, H, Nk, D = 1, 8, 8192, 128
    q = torch.randn((B, H, 1, D), generator=g).half()
    k = torch.randn((B, H, Nk, D), generator=g).half()
    v = torch.randn((B, H, Nk, D), generator=g).half()
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    sm = D ** -0.5
    a1 = M.attention_int8(*gpu(q8, k8, v, qs, ks), False, sm)
    a2 = M.attention_int8(*gpu(q8, k8, v, qs, ks), False, sm, num_splits="auto")
    assert max_abs(a2, a1) <= 1e-3
    f1 = M.attention_full_int8(*gpu(q8, k8, v8, qs, ks, vs), False, sm, p_round="rne")
    f2 = M.attention_full_int8(*gpu(q8, k8, v8, qs, ks, vs), False, sm, num_splits="auto", p_round="rne")
    assert max_abs(f2, f1) <= 2e-2 and max_abs(f2, _dense_cross(q, k, v, sm)) <= 3e-2


@pytest.mark.parametrize("Nq", [1, 3, 16])
def test_grouped_decoding_folds_heads_into_rows(Nq):
    """Grouped K/V heads with few queries: the wrapper runs a group's heads as rows of one head; every row's result must
    equal ordinary attention on repeated K/V, LSE included."""
    g_ = torch.Generator().manual_seed(72)
    B, H, Hkv, Nk, D = 2, 16, 4, 1500, 128
    q = torch.randn((B, H, Nq, D), generator=g_).half()
    k = torch.randn((B, Hkv, Nk, D), generator=g_).half()
    v = torch.randn((B, Hkv, Nk, D), generator=g_).half()
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    rep = lambda t: t.repeat_interleave(H // Hkv, dim=1)
    sm = D ** -0.5
    o, lse = M.attention(*gpu(q, k, v), False, sm, return_lse=True)
    exact = _dense_cross(q, rep(k), rep(v), sm)
    assert o.shape == (B, H, Nq, D) and max_abs(o, exact) <= 2e-3
    s = torch.matmul(q.float(), rep(k).float().transpose(2, 3)) * sm * 1.44269504
    assert (lse.cpu() - torch.logsumexp(s * 0.6931471805599453, dim=-1) * 1.44269504).abs().max().item() < 2e-3
    qd, kd = q8.float() * qs.float()[..., None], k8.float() * ks.float()[..., None]
    o = M.attention_int8(*gpu(q8, k8, v, qs, ks), False, sm, num_splits="auto")
    assert max_abs(o, _dense_cross(qd, rep(kd), rep(v), sm)) <= 3e-3
    o = M.attention_full_int8(*gpu(q8, k8, v8, qs, ks, vs), False, sm, p_round="rne")
    o_rep = M.attention_full_int8(*gpu(q8, rep(k8), rep(v8), qs, rep(ks), rep(vs)), False, sm, p_round="rne")     # ungrouped call
    assert torch.equal(o, o_rep)


@pytest.mark.parametrize("variant", ["full", "half", "fp"])
@pytest.mark.parametrize("Nq,Nk,D", [(128, 256, 64), (1, 300, 128), (37, 1000, 128), (200, 777, 64), (256, 384, 256), (65, 64 + 65, 128),
                                    (300, 130, 128)])
def test_causal_with_separate_lengths_is_aligned_bottom_right(variant, Nq, Nk, D):
    """A chunk of Nq new tokens against Nk cached keys: row i sees keys 0 .. i + Nk - Nq (csrc/mask.h:53,172 of the
    reference's CUDA tree); with fewer keys than queries the first Nq - Nk rows see nothing and come out as zeros."""
    B, H = 2, 2
    g = torch.Generator().manual_seed(45)
    q = torch.randn((B, H, Nq, D), generator=g).half()
    k = torch.randn((B, H, Nk, D), generator=g).half()
    v = torch.randn((B, H, Nk, D), generator=g).half()
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    sm = D ** -0.5
    if variant == "full":
        bn = M.block_n("full", D)
        o, lse = M.attention_full_int8(*gpu(q8, k8, v8, qs, ks, vs), True, sm, return_lse=True, p_round="rne")
        ref, lse_ref = O.attention_full_int8(q8, k8, v8, qs, ks, vs, True, sm, block_n=bn, p_requant=O.p_requant_rne, return_lse=True)
        torch.cuda.synchronize()
        if Nk >= Nq:
            assert_same_rounding(o, ref)
        else:
            assert max_abs(o, ref) <= MAX_ABS and mean_rel(o, ref) <= 2e-3
    elif variant == "half":
        o, lse = M.attention_int8(*gpu(q8, k8, v, qs, ks), True, sm, return_lse=True)
        ref, lse_ref = O.attention_int8(q8, k8, v, qs, ks, True, sm, block_n=64, return_lse=True)
        assert max_abs(o, ref) <= 4e-3 and mean_rel(o, ref) <= 5e-4
    else:
        o, lse = M.attention(*gpu(q, k, v), True, sm, return_lse=True)
        ref, lse_ref = O.attention_fp(q, k, v, True, sm, block_n=64, return_lse=True)
        assert max_abs(o, ref) <= 4e-3 and mean_rel(o, ref) <= 5e-4
    assert torch.isfinite(o).all()
    empty = max(Nq - Nk, 0)
    if empty:
        assert o[:, :, :empty].abs().max().item() == 0 and torch.isinf(lse[:, :, :empty]).all() and (lse[:, :, :empty] < 0).all()
    assert (lse.cpu()[:, :, empty:] - lse_ref[:, :, empty:]).abs().max().item() < 2e-3


@pytest.mark.parametrize("variant", ["full", "fp"])
def test_causal_separate_lengths_with_split_kv_and_per_batch_lengths(variant):
    B, H, Nq, Nk, D = 3, 2, 150, 900, 128
    lens = [900, 400, 150]
    g = torch.Generator().manual_seed(46)
    q = torch.randn((B, H, Nq, D), generator=g).half()
    k = torch.randn((B, H, Nk, D), generator=g).half()
    v = torch.randn((B, H, Nk, D), generator=g).half()
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    sm = D ** -0.5
    sl = torch.tensor(lens, dtype=torch.int32, device=DEV)
    if variant == "full":
        call = lambda **kw: M.attention_full_int8(*gpu(q8, k8, v8, qs, ks, vs), True, sm, seqlens_k=sl, p_round="rne", **kw)
        one = lambda b, n: O.attention_full_int8(q8[b:b + 1], k8[b:b + 1, :, :n], v8[b:b + 1, :, :n], qs[b:b + 1], ks[b:b + 1, :, :n],
                                                 vs[b:b + 1], True, sm, block_n=128, p_requant=O.p_requant_rne)
    else:
        call = lambda **kw: M.attention(*gpu(q, k, v), True, sm, seqlens_k=sl, **kw)
        one = lambda b, n: O.attention_fp(q[b:b + 1], k[b:b + 1, :, :n], v[b:b + 1, :, :n], True, sm, block_n=64)
    o = call()
    o3 = call(num_splits=3)
    torch.cuda.synchronize()
    for b, n in enumerate(lens):                       # every entry's mask is aligned to its own length
        ref = one(b, n)
        assert max_abs(o[b:b + 1], ref) <= 4e-3, (b, n)
        assert max_abs(o3[b:b + 1], ref) <= MAX_ABS and mean_rel(o3[b:b + 1], ref) <= 3e-2, (b, n)


@pytest.mark.parametrize("num_splits", [2, 4, "auto"])
@pytest.mark.parametrize("Nq", [2, 150])            # the decode-shaped kernel and the general one
def test_rows_without_a_key_on_the_split_path_give_zeros_and_minus_inf_lse(num_splits, Nq):
    """A batch entry whose cache is empty and (causal, fewer keys than queries) the rows above the first key: zeros and
    lse = -inf whether the call runs as one pass or as split partials merged by the combine kernel."""
    B, H, Nk, D = 3, 2, 1200, 128
    g = torch.Generator().manual_seed(47)
    q = torch.randn((B, H, Nq, D), generator=g).half()
    k = torch.randn((B, H, Nk, D), generator=g).half()
    v = torch.randn((B, H, Nk, D), generator=g).half()
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    sm = D ** -0.5
    lens = [1200, 0, 77]
    sl = torch.tensor(lens, dtype=torch.int32, device=DEV)
    for causal in (False, True):
        o, lse = M.attention_full_int8(*gpu(q8, k8, v8, qs, ks, vs), causal, sm, seqlens_k=sl, num_splits=num_splits,
                                       return_lse=True, p_round="rne")
        o1, lse1 = M.attention_full_int8(*gpu(q8, k8, v8, qs, ks, vs), causal, sm, seqlens_k=sl, return_lse=True, p_round="rne")
        torch.cuda.synchronize()
        assert torch.isfinite(o).all()
        assert o[1].abs().max().item() == 0 and torch.isinf(lse[1]).all() and (lse[1] < 0).all()
        if causal:                                     # entry 2 has 77 keys: rows 0 .. Nq - 78 see none of them
            empty = max(Nq - lens[2], 0)
            if empty:
                assert o[2, :, :empty].abs().max().item() == 0
                assert torch.isinf(lse[2, :, :empty]).all() and (lse[2, :, :empty] < 0).all()
            assert torch.isfinite(lse[2, :, empty:]).all()
        # the sign and the finite values agree with the single pass (the split frames differ in P8 only)
        assert torch.equal(torch.isinf(lse), torch.isinf(lse1)) and torch.equal(lse < 0, lse1 < 0)
        fin = torch.isfinite(lse1)
        assert (lse[fin] - lse1[fin]).abs().max().item() < 1e-3


# ------------------------------------------------------------------------------------------ grouped K/V heads
@pytest.mark.parametrize("variant", ["full", "half", "fp"])
@pytest.mark.parametrize("B,H,H_kv,N,D,causal", [(1, 8, 2, 256, 128, True), (2, 16, 16 // 4, 384, 64, False), (2, 4, 1, 256, 128, True)])
def test_grouped_kv_heads_equal_repeated_kv(variant, B, H, H_kv, N, D, causal):
    """k, v (and their scales) with fewer heads than q: query head h reads K/V head h // (H / H_kv), i.e. the result
    equals ordinary attention on K/V repeated along the head axis (the reference's CUDA tree has this form,
    csrc/flash_fwd_kernel_full_qi8.h:141; its Python API does not)."""
    g = H // H_kv
    q, _, _, _ = O.make_inputs(B, H, N, D, seed=50)
    _, k, v, _ = O.make_inputs(B, H_kv, N, D, seed=51)
    q8, qs = O.quant_pertoken(q)
    k8, ks = O.quant_pertoken(k)
    v8, vs = O.quant_pertensor(v)
    rep = lambda t: t.repeat_interleave(g, dim=1)
    sm = D ** -0.5
    if variant == "full":
        o = M.attention_full_int8(*gpu(q8, k8, v8, qs, ks, vs), causal, sm, p_round="rne")
        ref = O.attention_full_int8(q8, rep(k8), rep(v8), qs, rep(ks), rep(vs), causal, sm, block_n=M.block_n("full", D),
                                    p_requant=O.p_requant_rne)
        assert_same_rounding(o, ref)
    elif variant == "half":
        o = M.attention_int8(*gpu(q8, k8, v, qs, ks), causal, sm)
        ref = O.attention_int8(q8, rep(k8), rep(v), qs, rep(ks), causal, sm, block_n=64)
        assert max_abs(o, ref) <= 2e-3 and mean_rel(o, ref) <= 2e-4
    else:
        o = M.attention(*gpu(q, k, v), causal, sm)
        ref = O.attention_fp(q, rep(k), rep(v), causal, sm, block_n=64)
        assert max_abs(o, ref) <= 2e-3 and mean_rel(o, ref) <= 2e-4
    assert o.shape == (B, H, N, D)


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
    o = M.attention_full_int8(q8, k8, v8, qs, ks, vs, False, sm, p_round="rne")
    assert torch.isfinite(o).all()
    # every (batch, head) is independent: recomputing one slice alone gives the same bits
    for b, h in ((0, 0), (3, 31), (1, 17)):
        sl = lambda t: t[b:b + 1, h:h + 1].contiguous()
        o1 = M.attention_full_int8(sl(q8), sl(k8), sl(v8), sl(qs), sl(ks), sl(vs), False, sm, p_round="rne")
        assert torch.equal(o1, o[b:b + 1, h:h + 1])
    # the value scale is applied once, linearly: doubling it doubles the output exactly (power of two) wherever the
    # fp16 result is a normal number; subnormal results are rounded on a fixed 2^-24 grid and may differ by one step
    o2 = M.attention_full_int8(q8, k8, v8, qs, ks, vs * 2, False, sm, p_round="rne")
    normal = o.abs() > 2.0 ** -14
    assert torch.equal(o2[normal], (o * 2)[normal])
    assert (o2.float() - 2 * o.float()).abs().max().item() <= 2.0 ** -24
    # one slice against the CPU oracle at full sequence length
    b, h = 2, 5
    cpu = lambda t: t[b:b + 1, h:h + 1].cpu()
    ref = O.attention_full_int8(cpu(q8), cpu(k8), cpu(v8), cpu(qs), cpu(ks), cpu(vs), False, sm, block_n=128,
                                p_requant=O.p_requant_rne)
    assert max_abs(o[b:b + 1, h:h + 1], ref) <= 2e-3 and mean_rel(o[b:b + 1, h:h + 1], ref) <= 2e-4
    # the default (the reference's rounding of P) at the same size: same-rounding agreement with the oracle, and the
    # opt-in rounding stays inside the stated tolerance of the reference's result
    o_ref = M.attention_full_int8(q8, k8, v8, qs, ks, vs, False, sm)
    ref_r = O.attention_full_int8(cpu(q8), cpu(k8), cpu(v8), cpu(qs), cpu(ks), cpu(vs), False, sm, block_n=128)
    assert max_abs(o_ref[b:b + 1, h:h + 1], ref_r) <= 2e-3 and mean_rel(o_ref[b:b + 1, h:h + 1], ref_r) <= 2e-4
    assert max_abs(o[b:b + 1, h:h + 1], ref_r) <= 2e-2 and mean_rel(o[b:b + 1, h:h + 1], ref_r) <= 1e-2
    for bb, hh in ((0, 0), (3, 31)):
        sl = lambda t: t[bb:bb + 1, hh:hh + 1].contiguous()
        assert torch.equal(M.attention_full_int8(sl(q8), sl(k8), sl(v8), sl(qs), sl(ks), sl(vs), False, sm), o_ref[bb:bb + 1, hh:hh + 1])


@pytest.mark.parametrize("variant,B,H,H_kv,N,D,causal", [
    ("full", 1, 12, 12, 4096, 128, False),     # 12 heads: 8 dealt whole to the XCDs, the workgroups of 4 cut into 8 runs
    ("full", 3, 3, 3, 512, 64, True),          # 9 heads of 4 workgroups: the ninth is dealt one workgroup at a time
    ("full", 1, 20, 10, 256, 128, True),       # 10 K/V heads shared by 20 query heads
    ("full", 5, 1, 1, 300, 256, False),        # fewer heads than XCDs
    ("half", 1, 12, 12, 1024, 128, True),
    ("fp", 3, 5, 5, 640, 64, False),
])
def test_head_counts_that_do_not_divide_among_the_xcds(variant, B, H, H_kv, N, D, causal):
    """Whatever the workgroup -> (batch, head, query block) mapping of a launch, every output slice must be computed exactly
    once: the whole call reproduces, bit for bit, the calls on single (batch, K/V head) slices; one slice is also held
    against the oracle."""
    gen = torch.Generator(device=DEV).manual_seed(61)
    mk = lambda h: torch.randn((B, h, N, D), generator=gen, device=DEV, dtype=torch.float16)
    q, k, v = mk(H), mk(H_kv), mk(H_kv)
    sm, grp = D ** -0.5, H // H_kv
    if variant == "fp":
        args = (q, k, v)
        fn = lambda a: M.attention(*a, causal, sm)
    else:
        q8, qs = M.quant_pertoken(q)
        k8, ks = M.quant_pertoken(k)
        if variant == "half":
            args = (q8, k8, v, qs, ks)
            fn = lambda a: M.attention_int8(*a, causal, sm)
        else:
            v8, vs = M.quant_pertensor(v)
            args = (q8, k8, v8, qs, ks, vs)
            fn = lambda a: M.attention_full_int8(*a, causal, sm)
    o = fn(args)
    assert o.shape == (B, H, N, D) and torch.isfinite(o).all()
    for b in range(B):
        for hk in range(H_kv):
            sl = lambda i, t: (t[b:b + 1, hk * grp:(hk + 1) * grp] if i in ((0,) if variant == "fp" else (0, 3))
                               else t[b:b + 1, hk:hk + 1]).contiguous()
            o1 = fn(tuple(sl(i, t) for i, t in enumerate(args)))
            assert torch.equal(o1, o[b:b + 1, hk * grp:(hk + 1) * grp]), (b, hk)
    b, hk = B - 1, H_kv - 1
    h = hk * grp + grp - 1
    cq = lambda t: t[b:b + 1, h:h + 1].cpu()
    ck = lambda t: t[b:b + 1, hk:hk + 1].cpu()
    bn = M.block_n(variant, D)
    if variant == "fp":
        ref = O.attention_fp(cq(q), ck(k), ck(v), causal, sm, block_n=bn)
    elif variant == "half":
        ref = O.attention_int8(cq(q8), ck(k8), ck(v), cq(qs), ck(ks), causal, sm, block_n=bn)
    else:
        ref = O.attention_full_int8(cq(q8), ck(k8), ck(v8), cq(qs), ck(ks), ck(vs), causal, sm, block_n=bn)
    assert max_abs(o[b:b + 1, h:h + 1], ref) <= 4e-3 and mean_rel(o[b:b + 1, h:h + 1], ref) <= (2e-4 if variant == "full" else 6e-4)


def test_constant_v_gives_constant_columns_at_full_size():
    B, H, N, D = 2, 8, 4096, 128
    q8, k8, _, qs, ks, _ = _headline_inputs(B, H, N, D, seed=21)
    v8 = torch.full((B, H, N, D), 64, dtype=torch.int8, device=DEV)
    vs = torch.full((B, H), 1 / 64, dtype=torch.float16, device=DEV)
    o = M.attention_full_int8(q8, k8, v8, qs, ks, vs, True, D ** -0.5, p_round="rne")
    # O = sum(P8) / (127 l): the same for every column of a row.  Its distance from one is the mass P loses when it is
    # rounded to multiples of 1/127 (every p below 1/254 becomes zero): a property of the reference's quantisation
    # that grows with the number of keys, about 0.1 at 4096 keys with these inputs.
    assert torch.equal(o, o[..., :1].expand_as(o))
    assert (o.float() - 1).abs().max().item() < 0.25
    assert torch.equal(o[:, :, 0], torch.ones_like(o[:, :, 0]))    # row 0 sees key 0 only: P8 = 127, l = 1


@pytest.mark.parametrize("variant,B,H,N,D,causal", [
    ("full", 1, 32, 16384, 128, True),      # long-context prefill configuration
    ("half", 4, 32, 4096, 128, False),
    ("fp", 4, 32, 4096, 128, False),
    ("full", 4, 16, 4096, 256, False),      # head_dim 256 configuration
])
def test_other_benchmark_shapes_one_slice_against_oracle(variant, B, H, N, D, causal):
    g = torch.Generator(device=DEV).manual_seed(40)
    mk = lambda: torch.randn((B, H, N, D), generator=g, device=DEV, dtype=torch.float16)
    q, k, v = mk(), mk(), mk()
    sm = D ** -0.5
    b, h = B - 1, 7
    cpu = lambda t: t[b:b + 1, h:h + 1].cpu()
    bn = M.block_n(variant, D)
    if variant == "fp":
        o = M.attention(q, k, v, causal, sm)
        ref = O.attention_fp(cpu(q), cpu(k), cpu(v), causal, sm, block_n=bn)
    else:
        q8, qs = M.quant_pertoken(q)
        k8, ks = M.quant_pertoken(k)
        if variant == "half":
            o = M.attention_int8(q8, k8, v, qs, ks, causal, sm)
            ref = O.attention_int8(cpu(q8), cpu(k8), cpu(v), cpu(qs), cpu(ks), causal, sm, block_n=bn)
        else:
            v8, vs = M.quant_pertensor(v)
            o = M.attention_full_int8(q8, k8, v8, qs, ks, vs, causal, sm, p_round="rne")
            ref = O.attention_full_int8(cpu(q8), cpu(k8), cpu(v8), cpu(qs), cpu(ks), cpu(vs), causal, sm, block_n=bn,
                                        p_requant=O.p_requant_rne)
    assert torch.isfinite(o).all()
    # full-int8: the kernel and the oracle quantise the same P8 (only exp2 differs in the last place).  The 16-bit-P kernels
    # at head_dim <= 128 take exp2 against a reference point that lags the running maximum (the output is rescaled only
    # when a row's maximum rises by more than 8): the same p times a power-of-two-free factor, so its 16-bit rounding lands
    # elsewhere than the oracle's (relative 2^-12 per element, unbiased) - a few 1e-4 in the mean on outputs that are sums
    # of thousands of products with random signs, far inside the 1e-2 of the stated tolerance.
    tol_rel = 2e-4 if variant == "full" or D == 256 else 6e-4
    assert max_abs(o[b:b + 1, h:h + 1], ref) <= 4e-3 and mean_rel(o[b:b + 1, h:h + 1], ref) <= tol_rel


# ------------------------------------------------------------------------------------------ HIP graph capture
def test_forward_and_quantisers_replay_from_a_captured_graph():
    """The entry points only enqueue kernels (no allocation, no memset, no synchronisation of their own), so a caller
    can capture them in a HIP graph: replays interleaved with eager work must reproduce the eager results every time."""
    g = torch.Generator(device=DEV).manual_seed(80)
    B, H, N, D = 2, 4, 512, 128
    x = [torch.randn((B, H, N, D), generator=g, device=DEV, dtype=torch.float16) for _ in range(3)]
    sm = D ** -0.5

    def pipeline(q, k, v, splits):
        q8, qs = M.quant_pertoken(q)
        k8, ks = M.quant_pertoken(k)
        v8, vs = M.quant_pertensor(v)
        return M.attention_full_int8(q8, k8, v8, qs, ks, vs, True, sm, num_splits=splits, p_round="rne")

    for splits in (1, 3):
        static = [t.clone() for t in x]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):                       # warm-up outside the capture (library load, allocator pools)
            pipeline(*static, splits)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = pipeline(*static, splits)
        for rep in range(4):
            for t in static:                                # new inputs for every replay, written by eager kernels
                t.copy_(torch.randn(t.shape, generator=g, device=DEV, dtype=torch.float16))
            graph.replay()
            torch.cuda.synchronize()
            eager = pipeline(*static, splits)
            torch.cuda.synchronize()
            assert torch.equal(out, eager), (splits, rep)


@pytest.mark.parametrize("D,N,dtype", [(128, 2048, torch.float16), (64, 1024, torch.bfloat16), (128, 1000, torch.float16)])
def test_repeated_launches_are_bit_identical(D, N, dtype):
    """The output rows leave the kernel through LDS that held tiles a moment before (and into which the last block's
    empty copy slices still write): forty launches of one problem, many workgroups in flight, must agree bit for bit."""
    B, H = 4, 16
    g = torch.Generator(device=DEV).manual_seed(77)
    mk = lambda: torch.randn((B, H, N, D), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    q, k, v = mk(), mk(), mk()
    q8, qs = M.quant_pertoken(q)
    k8, ks = M.quant_pertoken(k)
    v8, vs = M.quant_pertensor(v)
    sm = D ** -0.5
    first = M.attention_full_int8(q8, k8, v8, qs, ks, vs, False, sm, out_dtype=dtype, p_round="rne")
    outs = [M.attention_full_int8(q8, k8, v8, qs, ks, vs, False, sm, out_dtype=dtype, p_round="rne") for _ in range(40)]
    torch.cuda.synchronize()
    assert torch.isfinite(first).all()
    for i, o in enumerate(outs):
        assert torch.equal(o, first), i
    b, h = 1, 3
    c = lambda t: t[b:b + 1, h:h + 1].cpu()
    ref = O.attention_full_int8(c(q8), c(k8), c(v8), c(qs), c(ks), c(vs), False, sm, block_n=M.block_n("full", D),
                                p_requant=O.p_requant_rne, out_dtype=dtype)
    assert max_abs(first[b:b + 1, h:h + 1], ref) <= (4e-3 if dtype == torch.float16 else 1.6e-2)
