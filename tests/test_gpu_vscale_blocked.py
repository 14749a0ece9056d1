"""GPU parity of the per-block, per-channel V scales (the V-scale layout of the reference's CUDA kernel,
csrc/flash_fwd_kernel_full_qi8.h:156-160, csrc/mask.h:313-340): the HIP quantiser bit for bit against the oracle's,
the forward against the oracle's blocked dequantisation at the kernel's key-block length, and the properties that
tie the blocked form to the scalar one."""
import pytest
import torch

import intfa_oracle as O
import int_flashattention_amd as M
from test_gpu_parity import DEV, MAX_ABS, MEAN_REL, assert_same_rounding, gpu, max_abs, mean_rel

pytestmark = pytest.mark.gpu


def blocked_inputs(B, H, N, D, seed, vsb, dtype=torch.float16, H_kv=None, burst=4.0):
    q, k, v, _ = O.make_inputs(B, H, N, D, seed=seed, dtype=dtype)
    if H_kv is not None:
        k, v = k[:, :H_kv].contiguous(), v[:, :H_kv].contiguous()
    if burst:                                                  # a burst in one channel of one key block
        v = v.clone(); v[:, :, N // 3: N // 3 + 40, D // 2] *= burst
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k)
    v8, vs = O.quant_perblock_channel(v, vsb)
    return dict(q=q, k=k, v=v, q8=q8, k8=k8, v8=v8, qs=qs, ks=ks, vs=vs)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,d,block", [(256, 128, 128), (300, 64, 64), (130, 256, 64), (77, 16, 128), (512, 32, 256)])
def test_quant_perblock_channel_bit_exact(dtype, N, d, block):
    g = torch.Generator().manual_seed(70 + d)
    x = (torch.randn((2, 3, N, d), generator=g) * 1.5).to(dtype)
    x[0, 1, : min(block, N), 3] = 0                            # an all-zero (block, channel): scale 0, zeros
    x[1, 2, N // 2, 5] = 60000 if dtype == torch.float16 else 3e30
    q_ref, s_ref = O.quant_perblock_channel(x, block)
    q, s = M.quant_perblock_channel(x.to(DEV), block)
    torch.cuda.synchronize()
    assert q.dtype == torch.int8 and s.dtype == torch.float32 and s.shape == s_ref.shape
    assert torch.equal(s.cpu(), s_ref)
    assert torch.equal(q.cpu(), q_ref)


def test_quant_perblock_channel_strided_input():
    g = torch.Generator().manual_seed(71)
    big = torch.randn((2, 2, 200, 256), generator=g).half()
    x = big[..., 64:192]                                       # row stride 256, offset keeps 16-byte alignment
    q_ref, s_ref = O.quant_perblock_channel(x.contiguous(), 128)
    q, s = M.quant_perblock_channel(big.to(DEV)[..., 64:192], 128)
    assert torch.equal(q.cpu(), q_ref) and torch.equal(s.cpu(), s_ref)


@pytest.mark.parametrize("B,H,N,D,causal,mult", [
    (1, 2, 512, 128, False, 1),
    (2, 2, 384, 64, True, 1),
    (1, 2, 512, 128, True, 2),         # one scale row per two key blocks of the kernel
    (1, 2, 256, 256, False, 1),        # head_dim 256: 64-key blocks, column halves
    (1, 2, 320, 256, True, 2),
    (1, 2, 384, 256, True, 1),         # three query blocks: one per workgroup, heaviest first
    (2, 3, 512, 256, True, 1),         # four query blocks: paired in one workgroup
    (1, 3, 300, 128, False, 1),        # ragged length: the last scale row covers 44 keys
    (1, 2, 97, 64, True, 1),
    # 64-key scale rows under the 128-key block: the granularity of the reference's CUDA kernel (kBlockN = 64 at
    # head_dim 128, csrc/flash_fwd_launch_template.h:514-519); P V is summed per 64-key half
    (1, 2, 512, 128, False, 0.5),
    (2, 2, 384, 64, True, 2),          # head_dim 64: 64-key blocks, one scale row per two of them
    (1, 3, 300, 128, True, 0.5),       # ragged: the last block holds 44 keys, its second scale row does not exist
    (1, 2, 200, 128, False, 0.5),      # the last block's second half holds 8 keys
    (1, 2, 160, 64, False, 1),         # head_dim 64: a scale row per 64-key block is the kernel's own block
    (1, 2, 40, 128, True, 0.5),        # few query rows (the decode-shaped kernel has no 64-key rows: the general one runs)
])
@pytest.mark.parametrize("p_round", ["rne", "reference"])
def test_blocked_v_scale_matches_oracle(B, H, N, D, causal, mult, p_round):
    bn = M.block_n("full", D)
    vsb = int(bn * mult)
    x = blocked_inputs(B, H, N, D, 80, vsb)
    sm = D ** -0.5
    o, lse = M.attention_full_int8(*gpu(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"]), causal, sm, p_round=p_round,
                                   v_scale_block=vsb, return_lse=True)
    torch.cuda.synchronize()
    assert o.dtype == torch.float16 and o.shape == (B, H, N, D)
    ref, lse_ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], causal, sm, block_n=bn,
                                         v_scale_block=vsb, return_lse=True)
    assert max_abs(o, ref) <= MAX_ABS and mean_rel(o, ref) <= MEAN_REL
    # every row's LSE (it does not depend on V or its scales; a row that lands in another row's slot shows here only)
    assert (lse.cpu() - lse_ref).abs().max().item() <= 1e-3
    same = ref if p_round == "reference" else O.attention_full_int8(
        x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], causal, sm, block_n=bn, v_scale_block=vsb,
        p_requant=O.p_requant_rne)
    assert_same_rounding(o, same)


def test_blocked_v_scale_filled_with_the_scalar_equals_the_scalar_entry():
    B, H, N, D = 1, 3, 384, 128
    q, k, v, _ = O.make_inputs(B, H, N, D, seed=81)
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    args = gpu(q8, k8, v8, qs, ks)
    want = M.attention_full_int8(*args, vs.to(DEV), True, 0.09, p_round="rne")
    vs4 = vs.float()[:, :, None, None].expand(B, H, 3, D).contiguous().to(DEV)
    got = M.attention_full_int8(*args, vs4, True, 0.09, p_round="rne")       # v_scale_block defaults to the kernel's key block
    torch.cuda.synchronize()
    # same products in another order (scale per block instead of once at the end): fp32 rounding only
    assert max_abs(got, want) <= 2e-3 and mean_rel(got, want) <= 1e-4


def test_blocked_v_scale_is_more_accurate_under_a_channel_burst():
    B, H, N, D = 1, 4, 1024, 128
    x = blocked_inputs(B, H, N, D, 82, 128, burst=25.0)
    sm = D ** -0.5
    exact = O.attention_exact(x["q"], x["k"], x["v"], False, sm).float()
    v8s, vss = O.quant_pertensor(x["v"])
    coarse = M.attention_full_int8(*gpu(x["q8"], x["k8"], v8s, x["qs"], x["ks"], vss), False, sm, p_round="rne").float().cpu()
    fine = M.attention_full_int8(*gpu(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"]), False, sm, p_round="rne").float().cpu()
    other = [c for c in range(D) if c != D // 2]
    err_c = (coarse - exact)[..., other].abs().mean().item()
    err_f = (fine - exact)[..., other].abs().mean().item()
    assert err_f < 0.5 * err_c


def test_blocked_v_scale_with_grouped_heads_split_kv_and_bf16():
    B, H, H_kv, N, D = 2, 8, 2, 640, 128
    x = blocked_inputs(B, H, N, D, 83, 128, dtype=torch.bfloat16, H_kv=H_kv)
    sm = D ** -0.5
    args = gpu(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"])
    one = M.attention_full_int8(*args, False, sm, out_dtype=torch.bfloat16, p_round="rne")
    rep = lambda t: t.repeat_interleave(H // H_kv, dim=1)
    ref = O.attention_full_int8(x["q8"], rep(x["k8"]), rep(x["v8"]), x["qs"], rep(x["ks"]), rep(x["vs"]), False, sm,
                                block_n=128, v_scale_block=128, p_requant=O.p_requant_rne, out_dtype=torch.bfloat16)
    assert one.dtype == torch.bfloat16
    d = (one.float().cpu() - ref.float()).abs()
    assert d.max().item() <= 3e-2 and mean_rel(one, ref) <= 3e-3          # bf16 output: 8-bit significand
    # split-KV: against the oracle evaluated with the same partition (a split restarts the running maximum, so its P is
    # quantised against another reference than in the single pass: the two differ by the P8 quantisation noise)
    split = M.attention_full_int8(*args, False, sm, out_dtype=torch.bfloat16, num_splits=3, p_round="reference")
    torch.cuda.synchronize()
    ref_split = O.attention_full_int8_splitkv(x["q8"], rep(x["k8"]), rep(x["v8"]), x["qs"], rep(x["ks"]), rep(x["vs"]), False,
                                              sm, 3, block_n=128, v_scale_block=128, out_dtype=torch.bfloat16)
    assert max_abs(split, ref_split) <= 3e-2 and mean_rel(split, ref_split) <= 3e-3
    assert max_abs(split, one) <= 4e-2 and mean_rel(split, one) <= 2e-2


def test_64_key_v_scale_rows_with_grouped_heads_split_kv_decode_shapes_and_bf16():
    B, H, H_kv, N, D = 2, 8, 2, 640, 128
    x = blocked_inputs(B, H, N, D, 85, 64, dtype=torch.bfloat16, H_kv=H_kv)
    sm = D ** -0.5
    args = gpu(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"])
    rep = lambda t: t.repeat_interleave(H // H_kv, dim=1)
    okw = dict(block_n=128, v_scale_block=64, out_dtype=torch.bfloat16)
    one = M.attention_full_int8(*args, True, sm, out_dtype=torch.bfloat16, v_scale_block=64, p_round="rne")
    ref = O.attention_full_int8(x["q8"], rep(x["k8"]), rep(x["v8"]), x["qs"], rep(x["ks"]), rep(x["vs"]), True, sm,
                                p_requant=O.p_requant_rne, **okw)
    assert max_abs(one, ref) <= 3e-2 and mean_rel(one, ref) <= 3e-3          # bf16 output: 8-bit significand
    split = M.attention_full_int8(*args, False, sm, out_dtype=torch.bfloat16, num_splits=3, p_round="reference", v_scale_block=64)
    ref_split = O.attention_full_int8_splitkv(x["q8"], rep(x["k8"]), rep(x["v8"]), x["qs"], rep(x["ks"]), rep(x["vs"]), False,
                                              sm, 3, **okw)
    assert max_abs(split, ref_split) <= 3e-2 and mean_rel(split, ref_split) <= 3e-3
    # decoding against the cache: three new tokens per head, grouped heads (no causal fold with 64-key rows), causal
    q3, qs3 = x["q8"][:, :, -3:].contiguous(), x["qs"][:, :, -3:].contiguous()
    dec = M.attention_full_int8(*gpu(q3, x["k8"], x["v8"], qs3, x["ks"], x["vs"]), True, sm, v_scale_block=64, p_round="rne")
    torch.cuda.synchronize()
    ref_dec = O.attention_full_int8(q3, rep(x["k8"]), rep(x["v8"]), qs3, rep(x["ks"]), rep(x["vs"]), True, sm,
                                    p_requant=O.p_requant_rne, block_n=128, v_scale_block=64)
    assert_same_rounding(dec, ref_dec)


def test_blocked_v_scale_small_head_dim_and_argument_checks():
    x = blocked_inputs(1, 2, 256, 32, 84, 128)
    o = M.attention_full_int8(*gpu(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"]), False, 0.2, v_scale_block=128, p_round="rne")
    ref = O.attention_full_int8(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"], False, 0.2, block_n=64,
                                v_scale_block=128, p_requant=O.p_requant_rne)
    assert_same_rounding(o, ref)
    with pytest.raises(RuntimeError):                          # 32 is not a multiple of the 64-key block
        v8, vs = O.quant_perblock_channel(x["v"], 32)
        M.attention_full_int8(*gpu(x["q8"], x["k8"], v8, x["qs"], x["ks"], vs), False, 0.2, v_scale_block=32, p_round="rne")
    with pytest.raises(RuntimeError):                          # neither is 96
        v8, vs = O.quant_perblock_channel(x["v"], 96)
        M.attention_full_int8(*gpu(x["q8"], x["k8"], v8, x["qs"], x["ks"], vs), False, 0.2, v_scale_block=96, p_round="rne")
    with pytest.raises(ValueError):                            # wrong number of scale rows
        M.attention_full_int8(*gpu(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"][:, :, :1]), False, 0.2, v_scale_block=128, p_round="rne")
    with pytest.raises(ValueError):
        M.attention_full_int8(*gpu(x["q8"], x["k8"], x["v8"], x["qs"], x["ks"], x["vs"][:, :, 0, 0]), False, 0.2, v_scale_block=128, p_round="rne")


def test_quant_perblock_channel_bit_exact_on_many_magnitudes():
    """2 M elements whose columns span eight orders of magnitude: the reciprocal-based quotient of the kernel must round
    like the oracle's division everywhere (ties included: multiples of 1/254 of a column maximum are planted)."""
    g = torch.Generator().manual_seed(72)
    x = torch.randn((2, 2, 4096, 128), generator=g)
    x = x * torch.pow(10.0, torch.rand((1, 1, 1, 128), generator=g) * 8 - 5)
    x = x.half()
    col_max = x[:, :, :128].abs().amax(dim=2, keepdim=True).float()
    ties = (torch.arange(128).view(1, 1, 128, 1).float() + 0.5) / 127.0 * col_max        # exact .5 quotients where representable
    x[:, :, 1:129:2] = ties[:, :, 1::2].half()
    q_ref, s_ref = O.quant_perblock_channel(x, 128)
    q, s = M.quant_perblock_channel(x.to(DEV), 128)
    torch.cuda.synchronize()
    assert torch.equal(s.cpu(), s_ref)
    assert torch.equal(q.cpu(), q_ref)
