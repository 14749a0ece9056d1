"""The C ABI from a caller that is not Python: tests/capi_c/intfa_c_caller.c (plain C, gcc, the HIP runtime for device
memory) runs intfa_fwd_full_int8 on tensors handed over in a file; its output must be the wrapper's, bit for bit."""
import os
import subprocess

import numpy as np
import pytest
import torch

import intfa_oracle as O
import int_flashattention_amd as M
from int_flashattention_amd import build as B

pytestmark = pytest.mark.gpu


def _caller():
    if not os.path.exists(B.C_CALLER):
        B.build_c_caller(verbose=False)
    return B.C_CALLER


@pytest.mark.parametrize("Bz,H,N,D,causal,splits", [(2, 3, 384, 128, False, 1), (1, 2, 512, 64, True, 1), (1, 4, 1000, 128, False, 3)])
def test_c_caller_output_equals_the_python_wrappers(tmp_path, Bz, H, N, D, causal, splits):
    q, k, v, _ = O.make_inputs(Bz, H, N, D, seed=40)
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    fin, fout = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(fin, "wb") as f:
        for t in (q8, k8, v8):
            f.write(t.contiguous().numpy().tobytes())
        for t in (qs, ks, vs):
            f.write(t.contiguous().view(torch.int16).numpy().tobytes())
    r = subprocess.run([_caller(), fin, fout, str(Bz), str(H), str(N), str(D), str(int(causal)), str(splits)],
                       capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stderr
    assert r.stdout.startswith("ok") and r.stdout.strip().endswith(f"block_n {M.block_n('full', D)}")
    got = torch.from_numpy(np.fromfile(fout, dtype=np.float16).reshape(Bz, H, N, D))
    dev = "cuda"
    want = M.attention_full_int8(q8.to(dev), k8.to(dev), v8.to(dev), qs.to(dev), ks.to(dev), vs.to(dev), causal, D ** -0.5,
                                 num_splits=splits, p_round="rne")
    torch.cuda.synchronize()
    assert torch.equal(got, want.cpu())


def test_c_caller_reports_rejected_arguments(tmp_path):
    fin = str(tmp_path / "in.bin")
    open(fin, "wb").write(bytes(3 * 2 * 128 * 96 + 2 * 2 * 128 * 2 + 2 * 2))
    r = subprocess.run([_caller(), fin, str(tmp_path / "out.bin"), "1", "2", "128", "96", "0", "1"], capture_output=True, text=True,
                       timeout=100)
    assert r.returncode == 5 and "head_dim" in r.stderr
