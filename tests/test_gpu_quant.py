"""GPU tests of the HIP quantisers (C ABI: intfa_quant_pertoken / intfa_quant_pertensor) against the CPU oracle's
restatement of benchmark.py:96-107.  Integer outputs and scales must be bit-exact."""
import pytest
import torch

import intfa_oracle as O
import int_flashattention_amd as M

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _check(x):
    q_t, s_t = M.quant_pertoken(x.to(DEV))
    q_r, s_r = O.quant_pertoken(x)
    assert q_t.dtype == torch.int8 and s_t.dtype == x.dtype and q_t.is_contiguous()
    assert torch.equal(s_t.cpu(), s_r)
    assert torch.equal(q_t.cpu(), q_r)
    q_t, s_t = M.quant_pertensor(x.to(DEV))
    q_r, s_r = O.quant_pertensor(x)
    assert s_t.shape == x.shape[:2] and torch.equal(s_t.cpu(), s_r)
    assert torch.equal(q_t.cpu(), q_r)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("d", [16, 32, 64, 128, 256])
def test_quantisers_bit_exact_random(dtype, d):
    g = torch.Generator().manual_seed(100 + d)
    for std in (1.0, 0.5, 7.3):
        x = (torch.randn((2, 3, 200, d), generator=g) * std).to(dtype)
        _check(x)


def test_quantisers_ties_and_extremes():
    """Hand-made rows: exact .5 quotients (round-half-even), a row whose maximum is negative, tiny and huge magnitudes."""
    d = 16
    rows = []
    base = torch.zeros(d)
    base[0] = 127.0                       # scale exactly 1: quotients equal the values
    base[1:9] = torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5])
    rows.append(base)
    neg = -torch.arange(1, d + 1, dtype=torch.float32) * 3.25
    rows.append(neg)
    rows.append(torch.full((d,), 6.0e-5))             # fp16 subnormal range for the scale
    rows.append(torch.linspace(-60000, 60000, d))
    rows.append(torch.tensor([1.0, -1.0] * (d // 2)) * 0.33)
    x = torch.stack(rows)[None, None].contiguous()    # [1, 1, 5, 16]
    _check(x.half())
    _check(x.bfloat16())


def test_quantisers_strided_input_and_odd_sizes():
    g = torch.Generator().manual_seed(7)
    x = torch.randn((2, 77, 5, 64), generator=g).half()          # stored [B, N, H, d]
    xv = x.permute(0, 2, 1, 3)                                    # viewed [B, H, N, d]
    q_t, s_t = M.quant_pertoken(x.to(DEV).permute(0, 2, 1, 3))
    q_r, s_r = O.quant_pertoken(xv)
    assert torch.equal(q_t.cpu(), q_r) and torch.equal(s_t.cpu(), s_r)
    q_t, s_t = M.quant_pertensor(x.to(DEV).permute(0, 2, 1, 3))
    q_r, s_r = O.quant_pertensor(xv)
    assert torch.equal(q_t.cpu(), q_r) and torch.equal(s_t.cpu(), s_r)


def test_quantisers_full_size_properties():
    """Benchmark shape: every row reaches +-127 (up to the rounding of the scale), |q| <= 127 in fp16, the dequantised
    value is within half a step of the input, and a slice equals the oracle."""
    B, H, N, D = 4, 32, 4096, 128
    g = torch.Generator(device=DEV).manual_seed(3)
    x = torch.randn((B, H, N, D), generator=g, device=DEV, dtype=torch.float16)
    q, s = M.quant_pertoken(x)
    assert q.abs().amax(dim=-1).min().item() == 127 and q.abs().max().item() == 127
    err = (q.float() * s.float()[..., None] - x.float()).abs()
    # half a step, plus the fp16 rounding of the quotient itself (ulp 1/16 at 64..127) before it is rounded to an integer
    assert (err <= (0.5 + 1.0 / 32 + 1e-3) * s.float()[..., None] + 1e-6).all()
    qv, sv = M.quant_pertensor(x)
    assert qv.abs().amax(dim=(-2, -1)).min().item() == 127
    b, h = 3, 17
    q_r, s_r = O.quant_pertoken(x[b:b + 1, h:h + 1].cpu())
    assert torch.equal(q[b:b + 1, h:h + 1].cpu(), q_r) and torch.equal(s[b:b + 1, h:h + 1].cpu(), s_r)
    q_r, s_r = O.quant_pertensor(x[b:b + 1, h:h + 1].cpu())
    assert torch.equal(qv[b:b + 1, h:h + 1].cpu(), q_r) and torch.equal(sv[b:b + 1, h:h + 1].cpu(), s_r)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_quantisers_every_16bit_value_against_many_scales(dtype):
    """Every finite value of the 16-bit type divided by 96 different row scales: the kernels form the quotient from a
    reciprocal with a correction step, which must round exactly like the oracle's division."""
    bits = torch.arange(0, 1 << 16, dtype=torch.int32)
    allv = bits.to(torch.int16).view(dtype)
    allv = allv[torch.isfinite(allv.float())]
    g = torch.Generator().manual_seed(99)
    maxima = torch.cat([torch.tensor([127.0, 1.0, 0.33, 6.0e-5, 60000.0, 3.0, 2.0 ** -10, 1.5, 0.999, 254.0]),
                        torch.rand(86, generator=g) * 8 + 0.01]).to(dtype)
    rows = []
    for m in maxima:
        vals = allv[allv.float().abs() <= m.float().abs()]
        pad = (-vals.numel()) % 15
        vals = torch.cat([vals, vals[:pad]])
        block = torch.cat([m.expand(vals.numel() // 15, 1), vals.view(-1, 15)], dim=1)      # the maximum leads every row
        rows.append(block)
    x = torch.cat(rows)[None, None].contiguous()                                           # [1, 1, R, 16]
    q_t, s_t = M.quant_pertoken(x.to(DEV))
    q_r, s_r = O.quant_pertoken(x)
    assert torch.equal(s_t.cpu(), s_r)
    assert torch.equal(q_t.cpu(), q_r)
