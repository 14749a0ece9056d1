"""Seeded random sweeps over shapes and options of the three forward entry points, through the C ABI, against the CPU
oracle.  The fixed-shape tests pin named cases; these draw the combinations nobody thought of: head dims 16-256, ragged
query and key lengths on either side of every tile size, grouped K/V heads, per-batch cache lengths, both P roundings,
all output and scale types, blocked V scales, split counts, the causal mask with more or fewer queries than keys.  A case
is a pure function of its seed (printed in the test id).  Outputs, every row's log-sum-exp and the rows that see no key
are checked.

Bounds (mean-rel = mean|a-b| / mean|b|):
  full-int8, single pass, against the oracle at the kernel's key block and rounding: fp16 out max-abs 2e-2 / mean-rel
  2e-3 (one P8 step next to a rounding boundary moves an output by up to 1/127 of a V value), bf16 out 3e-2 / 5e-3;
  with fewer than 64 keys a single flipped P8 step weighs more: 3e-2 / 1e-2.
  full-int8, split-KV against the SINGLE-PASS oracle: 6e-2 / 4e-2 - a split requantises P relative to its own running
  maximum, so its P8 values differ from the single pass's, most with a sharp softmax (sm_scale 0.3) where few P8 steps
  carry the row (the same-split oracle comparison, with the single-pass bounds, is in test_gpu_parity.py and
  test_gpu_decode.py).
  half-int8 and fp16/bf16 (no requantisation): fp16 4e-3 / 6e-4, bf16 3e-2 / 3e-3.
  LSE: 4e-3 absolute on rows that see a key; rows that see none give zeros and lse = -inf.
"""
import random

import pytest
import torch

import intfa_oracle as O
import int_flashattention_amd as M

pytestmark = pytest.mark.gpu
DEV = "cuda"


def errs(a, b):
    a, b = a.float().cpu(), b.float().cpu()
    return (a - b).abs().max().item(), ((a - b).abs().mean() / b.abs().mean().clamp_min(1e-9)).item()


def check_rows(o, lse, ref, lref, tol, tag):
    """o, ref: [1, H, Nq, D]; lse, lref: [1, H, Nq].  Rows whose oracle lse is -inf see no key."""
    seen = torch.isfinite(lref)
    l = lse.cpu()
    assert torch.equal(torch.isfinite(l), seen), f"{tag}: rows without a key differ"
    assert bool(torch.isfinite(o).all()), f"{tag}: non-finite output"
    if (~seen).any():
        assert o.cpu()[~seen].abs().max().item() == 0, f"{tag}: a row without keys is not zero"
        assert bool((l[~seen] < 0).all()), f"{tag}: lse of a row without keys is not -inf"
    if seen.any():
        ma, mr = errs(o.cpu()[seen], ref[seen])
        le = (l[seen] - lref[seen]).abs().max().item()
        assert ma <= tol[0] and mr <= tol[1], f"{tag}: max_abs {ma:.3g} mean_rel {mr:.3g} (bounds {tol})"
        assert le < 4e-3, f"{tag}: lse differs by {le:.3g}"


def draw_lengths(rng, B, Nk, allow_empty):
    choices = [Nk, max(1, Nk // 2), max(1, Nk - 1), max(1, Nk - 3), 1] + ([0] if allow_empty else [])
    return [rng.choice(choices) for _ in range(B)]


# ---------------------------------------------------------------------------------------------------------------------
# full-int8: general and decode-shaped calls
# ---------------------------------------------------------------------------------------------------------------------
def full_int8_case(seed):
    rng = random.Random(seed)
    decode = rng.random() < 0.5
    D = rng.choice([16, 32, 64, 128, 256])
    B = rng.choice([1, 2, 3])
    Hkv = rng.choice([1, 2, 3])
    g = rng.choice([1, 1, 2, 4, 8] if decode else [1, 1, 2, 4])
    if decode:
        Nq = rng.choice([1, 1, 2, 5, 16, 31, 32, 33, 64, 65, 100])
        Nk = rng.choice([1, 50, 128, 129, 500, 1024, 1500, 3000])
    else:
        Nq = rng.choice([1, 5, 31, 64, 65, 128, 129, 200, 256, 300, 511, 777])
        Nk = rng.choice([Nq, Nq, 1, 50, 128, 129, 256, 300, 500, 1000, 1500])
    pr = rng.choice(["rne", "reference"])
    odt = rng.choice([torch.float16, torch.bfloat16])
    sdt = rng.choice([torch.float16, torch.float32, torch.bfloat16])
    splits = rng.choice([1, 1, 2, 4, "auto"])
    bn = M.block_n("full", D)
    vb = rng.choice([None, None, bn, 2 * bn])
    if vb and bn == 128 and rng.random() < 0.3:
        vb = 64                                             # V scale rows of 64 keys (two per 128-key block)
    causal = rng.random() < 0.5
    use_len = rng.random() < 0.4
    sm = rng.choice([D ** -0.5, 0.05, 0.3])
    lens = draw_lengths(rng, B, Nk, allow_empty=True) if use_len else None
    return dict(D=D, B=B, Hkv=Hkv, g=g, Nq=Nq, Nk=Nk, pr=pr, odt=odt, sdt=sdt, splits=splits, vb=vb, causal=causal,
                lens=lens, sm=sm, bn=bn)


@pytest.mark.parametrize("seed", range(1000, 1090))
def test_full_int8_random_case(seed):
    c = full_int8_case(seed)
    B, Hkv, g, Nq, Nk, D, vb = c["B"], c["Hkv"], c["g"], c["Nq"], c["Nk"], c["D"], c["vb"]
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn((B, Hkv * g, Nq, D), generator=gen).half()
    k = torch.randn((B, Hkv, Nk, D), generator=gen).half()
    v = torch.randn((B, Hkv, Nk, D), generator=gen).half()
    q8, qs = O.quant_pertoken(q)
    k8, ks = O.quant_pertoken(k)
    v8, vs = O.quant_perblock_channel(v, vb) if vb else O.quant_pertensor(v)
    qs, ks = qs.to(c["sdt"]), ks.to(c["sdt"])
    if not vb:
        vs = vs.to(c["sdt"])
    kw = dict(num_splits=c["splits"], p_round=c["pr"], out_dtype=c["odt"], return_lse=True)
    if vb:
        kw["v_scale_block"] = vb
    if c["lens"]:
        kw["seqlens_k"] = torch.tensor(c["lens"], dtype=torch.int32, device=DEV)
    o, lse = M.attention_full_int8(q8.to(DEV), k8.to(DEV), v8.to(DEV), qs.to(DEV), ks.to(DEV), vs.to(DEV), c["causal"], c["sm"], **kw)
    torch.cuda.synchronize()
    rq = O.p_requant_rne if c["pr"] == "rne" else O.p_requant_reference
    rep = lambda t: t.repeat_interleave(g, dim=1)
    for b in range(B):
        n = c["lens"][b] if c["lens"] else Nk
        tag = f"seed {seed} {c} batch {b} n={n}"
        if n == 0:
            assert o[b].abs().max().item() == 0 and bool((lse[b] < 0).all()) and bool(torch.isinf(lse[b]).all()), tag
            continue
        s = lambda t: t[b:b + 1]
        okw = dict(v_scale_block=vb) if vb else {}
        vsb = s(rep(vs))[:, :, :(n + vb - 1) // vb] if vb else s(rep(vs))
        ref, lref = O.attention_full_int8(s(q8), s(rep(k8))[:, :, :n], s(rep(v8))[:, :, :n], s(qs), s(rep(ks))[:, :, :n], vsb,
                                          c["causal"], c["sm"], block_n=c["bn"], p_requant=rq, out_dtype=c["odt"], return_lse=True, **okw)
        tol = (2e-2, 2e-3) if c["splits"] == 1 else (6e-2, 4e-2)
        if c["odt"] == torch.bfloat16:
            tol = (max(tol[0], 3e-2), max(tol[1], 5e-3))
        if n < 64:
            tol = (max(tol[0], 3e-2), max(tol[1], 1e-2))
        check_rows(o[b:b + 1], lse[b:b + 1], ref, lref, tol, tag)


# ---------------------------------------------------------------------------------------------------------------------
# half-int8 and fp16/bf16: general, head_dim 256 and decode-shaped calls
# ---------------------------------------------------------------------------------------------------------------------
def f16pv_case(seed):
    rng = random.Random(seed)
    variant = rng.choice(["half", "fp"])
    decode = rng.random() < 0.4
    D = rng.choice([16, 32, 64, 128, 256, 256])
    B = rng.choice([1, 2, 3])
    Hkv = rng.choice([1, 2, 3])
    g = rng.choice([1, 1, 2, 4])
    if decode:
        Nq = rng.choice([1, 1, 2, 5, 16, 31, 32, 33, 64, 65])
        Nk = rng.choice([1, 50, 64, 65, 128, 129, 500, 1024, 1500, 3000])
    else:
        Nq = rng.choice([1, 31, 64, 65, 100, 128, 129, 200, 256, 300, 384, 500, 640])
        Nk = rng.choice([Nq, Nq, 1, 50, 63, 64, 65, 128, 129, 191, 192, 500, 640, 1024, 1500])
    dt = rng.choice([torch.float16, torch.bfloat16])
    sdt = rng.choice([torch.float16, torch.float32, torch.bfloat16])
    splits = rng.choice([1, 1, 2, 4, "auto"])
    causal = rng.random() < 0.5
    use_len = rng.random() < 0.4
    sm = rng.choice([D ** -0.5, 0.05, 0.2])
    lens = draw_lengths(rng, B, Nk, allow_empty=False) if use_len else None
    return dict(variant=variant, D=D, B=B, Hkv=Hkv, g=g, Nq=Nq, Nk=Nk, dt=dt, sdt=sdt, splits=splits, causal=causal, lens=lens, sm=sm)


@pytest.mark.parametrize("seed", range(2000, 2090))
def test_half_int8_and_fp_random_case(seed):
    c = f16pv_case(seed)
    B, Hkv, g, Nq, Nk, D, dt = c["B"], c["Hkv"], c["g"], c["Nq"], c["Nk"], c["D"], c["dt"]
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn((B, Hkv * g, Nq, D), generator=gen).to(dt)
    k = torch.randn((B, Hkv, Nk, D), generator=gen).to(dt)
    v = torch.randn((B, Hkv, Nk, D), generator=gen).to(dt)
    kw = dict(num_splits=c["splits"], return_lse=True)
    if c["lens"]:
        kw["seqlens_k"] = torch.tensor(c["lens"], dtype=torch.int32, device=DEV)
    if c["variant"] == "half":
        q8, qs = O.quant_pertoken(q)
        k8, ks = O.quant_pertoken(k)
        qs, ks = qs.to(c["sdt"]), ks.to(c["sdt"])
        o, lse = M.attention_int8(q8.to(DEV), k8.to(DEV), v.to(DEV), qs.to(DEV), ks.to(DEV), c["causal"], c["sm"], **kw)
    else:
        o, lse = M.attention(q.to(DEV), k.to(DEV), v.to(DEV), c["causal"], c["sm"], **kw)
    torch.cuda.synchronize()
    rep = lambda t: t.repeat_interleave(g, dim=1)
    for b in range(B):
        n = c["lens"][b] if c["lens"] else Nk
        tag = f"seed {seed} {c} batch {b} n={n}"
        s = lambda t: t[b:b + 1]
        if c["variant"] == "half":
            ref, lref = O.attention_int8(s(q8), s(rep(k8))[:, :, :n], s(rep(v))[:, :, :n], s(qs), s(rep(ks))[:, :, :n], c["causal"], c["sm"],
                                         block_n=64, out_dtype=dt, return_lse=True)
        else:
            ref, lref = O.attention_fp(s(q), s(rep(k))[:, :, :n], s(rep(v))[:, :, :n], c["causal"], c["sm"], block_n=64, return_lse=True)
        tol = (4e-3, 6e-4) if dt == torch.float16 else (3e-2, 3e-3)
        check_rows(o[b:b + 1], lse[b:b + 1], ref, lref, tol, tag)
