"""The committed fixtures of tests/golden (made by tests/golden/make_golden.py from the CPU oracle): the oracle must still
reproduce them bit for bit (CPU), and the kernels must match them within the stated tolerances (GPU)."""
import os

import numpy as np
import pytest
import torch

import intfa_oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attention_small.npz")


def _load():
    z = np.load(GOLD, allow_pickle=False)
    return {k: torch.from_numpy(z[k]) if z[k].shape else float(z[k]) for k in z.files}


def test_oracle_reproduces_the_fixtures():
    g = _load()
    sm = g["sm_scale"]
    q8, qs = O.quant_pertoken(g["q"]); k8, ks = O.quant_pertoken(g["k"]); v8, vs = O.quant_pertensor(g["v"])
    assert torch.equal(q8, g["q8"]) and torch.equal(k8, g["k8"]) and torch.equal(v8, g["v8"])
    assert torch.equal(qs, g["qs"]) and torch.equal(ks, g["ks"]) and torch.equal(vs, g["vs"])
    assert torch.equal(O.qk_int32(q8, k8), g["s_int32"])
    for causal, tag in ((False, "dense"), (True, "causal")):
        assert torch.equal(O.attention_full_int8(q8, k8, v8, qs, ks, vs, causal, sm, block_n=64), g[f"full_ref_{tag}"])
        assert torch.equal(O.attention_full_int8(q8, k8, v8, qs, ks, vs, causal, sm, block_n=64, p_requant=O.p_requant_rne),
                           g[f"full_rne_{tag}"])
        assert torch.equal(O.attention_int8(q8, k8, g["v"], qs, ks, causal, sm, block_n=64), g[f"half_{tag}"])
        assert torch.equal(O.attention_fp(g["q"], g["k"], g["v"], causal, sm, block_n=64), g[f"fp_{tag}"])


@pytest.mark.gpu
def test_kernels_match_the_fixtures():
    import int_flashattention_amd as M
    g = _load()
    sm = g["sm_scale"]
    dev = "cuda"
    c = lambda *names: [g[n].to(dev) for n in names]
    q8, qs = M.quant_pertoken(g["q"].to(dev))
    v8, vs = M.quant_pertensor(g["v"].to(dev))
    assert torch.equal(q8.cpu(), g["q8"]) and torch.equal(qs.cpu(), g["qs"])
    assert torch.equal(v8.cpu(), g["v8"]) and torch.equal(vs.cpu(), g["vs"])
    assert torch.equal(M.debug_qk_int32(*c("q8", "k8")).cpu(), g["s_int32"])
    err = lambda a, b: ((a.float().cpu() - b.float()).abs().max().item(),
                        ((a.float().cpu() - b.float()).abs().mean() / b.float().abs().mean()).item())
    for causal, tag in ((False, "dense"), (True, "causal")):
        o = M.attention_full_int8(*c("q8", "k8", "v8", "qs", "ks", "vs"), causal, sm, p_round="reference")
        ma, mr = err(o, g[f"full_ref_{tag}"]); assert ma <= 8e-3 and mr <= 2e-4
        o = M.attention_full_int8(*c("q8", "k8", "v8", "qs", "ks", "vs"), causal, sm, p_round="rne")
        ma, mr = err(o, g[f"full_rne_{tag}"]); assert ma <= 8e-3 and mr <= 2e-4
        ma, mr = err(o, g[f"full_ref_{tag}"]); assert ma <= 2e-2 and mr <= 1e-2       # the stated tolerance
        o = M.attention_int8(*c("q8", "k8", "v", "qs", "ks"), causal, sm)
        ma, mr = err(o, g[f"half_{tag}"]); assert ma <= 2e-3 and mr <= 3e-4
        o = M.attention(*c("q", "k", "v"), causal, sm)
        ma, mr = err(o, g[f"fp_{tag}"]); assert ma <= 2e-3 and mr <= 3e-4
