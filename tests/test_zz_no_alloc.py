"""intfa_fwd_full_int8_static - the entry point for callers that cannot allocate device memory - against
intfa_fwd_full_int8 with a caller-provided workspace: same bits, on two calls in a row (the second on a smaller problem,
so stale partials of the first call lie behind it in the library's scratch array), and the size limit is enforced.
Both entry points are called through the C ABI (ctypes), exactly as a C caller would."""
import ctypes

import pytest
import torch

import intfa_oracle as O
from int_flashattention_amd import _capi

pytestmark = pytest.mark.gpu
DEV = "cuda"


def make_problem(B, H, Nq, Nk, D, seed, causal):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((B, H, Nq, D), generator=g).half()
    k = torch.randn((B, H, Nk, D), generator=g).half()
    v = torch.randn((B, H, Nk, D), generator=g).half()
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    t = [x.to(DEV) for x in (q8, k8, v8, qs, ks, vs)]
    return dict(t=t, B=B, H=H, Nq=Nq, Nk=Nk, D=D, causal=causal, cpu=(q8, k8, v8, qs, ks, vs))


def fill(pb, out, lse, num_splits):
    q8, k8, v8, qs, ks, vs = pb["t"]
    p = _capi.FwdParams()
    p.q, p.k, p.v, p.out, p.lse = q8.data_ptr(), k8.data_ptr(), v8.data_ptr(), out.data_ptr(), lse.data_ptr()
    p.q_scale, p.k_scale, p.v_scale = qs.data_ptr(), ks.data_ptr(), vs.data_ptr()
    for name, t in (("q", q8), ("k", k8), ("v", v8), ("o", out)):
        setattr(p, f"{name}_stride_b", t.stride(0)); setattr(p, f"{name}_stride_h", t.stride(1)); setattr(p, f"{name}_stride_n", t.stride(2))
    p.qs_stride_b, p.qs_stride_h, p.qs_stride_n = qs.stride()
    p.ks_stride_b, p.ks_stride_h, p.ks_stride_n = ks.stride()
    p.vs_stride_b, p.vs_stride_h = vs.stride()
    p.batch, p.heads, p.seqlen, p.seqlen_k, p.head_dim = pb["B"], pb["H"], pb["Nq"], pb["Nk"], pb["D"]
    p.scale_dtype, p.io_dtype = _capi.INTFA_F16, _capi.INTFA_F16
    p.causal, p.sm_scale, p.p_round, p.num_splits = int(pb["causal"]), pb["D"] ** -0.5, _capi.PROUND_REFERENCE, num_splits
    return p


def run_both(pb, num_splits):
    lib = _capi.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    shape = (pb["B"], pb["H"], pb["Nq"], pb["D"])
    outs = []
    for static in (False, True):
        out = torch.full(shape, float("nan"), dtype=torch.float16, device=DEV)
        lse = torch.full(shape[:3], float("nan"), dtype=torch.float32, device=DEV)
        p = fill(pb, out, lse, num_splits)
        if static:
            p.workspace, p.workspace_bytes = None, 0          # ignored anyway
            rc = lib.intfa_fwd_full_int8_static(ctypes.byref(p), stream)
        else:
            need = lib.intfa_fwd_workspace_bytes(ctypes.byref(p))
            ws = torch.empty((max(need, 16),), dtype=torch.uint8, device=DEV)
            p.workspace, p.workspace_bytes = ws.data_ptr(), need
            rc = lib.intfa_fwd_full_int8(ctypes.byref(p), stream)
        assert rc == 0, lib.intfa_error_string(rc)
        torch.cuda.synchronize()
        outs.append((out, lse))
    return outs


def test_static_scratch_entry_point_equals_the_workspace_entry_point_on_two_calls_in_a_row():
    big = make_problem(2, 4, 256, 2048, 128, seed=901, causal=True)       # general kernel, 4 splits: 4 MiB of partials
    small = make_problem(1, 2, 3, 700, 64, seed=902, causal=False)        # decode-shaped kernel, ragged cache, 3 splits
    for pb, splits in ((big, 4), (small, 3)):
        (o_ws, lse_ws), (o_st, lse_st) = run_both(pb, splits)
        assert torch.isfinite(o_st).all() and torch.isfinite(lse_st).all()
        assert torch.equal(o_st, o_ws) and torch.equal(lse_st, lse_ws)
        # and both are the oracle's split evaluation (reference rounding) where the oracle has one (equal lengths or not causal)
        if not pb["causal"]:
            ref = O.attention_full_int8_splitkv(*pb["cpu"], False, pb["D"] ** -0.5, splits, block_n=64 if pb["D"] != 128 else 128)
            assert (o_st.float().cpu() - ref.float()).abs().max().item() <= 2e-2
    # a single pass needs no scratch at all and is the plain entry point
    (o_ws, lse_ws), (o_st, lse_st) = run_both(small, 1)
    assert torch.equal(o_st, o_ws) and torch.equal(lse_st, lse_ws)


def test_static_scratch_entry_point_records_into_a_graph():
    """After its first call on a device the entry point allocates, frees and synchronises nothing: a stream capture, which
    any of those would break, records it (forward and combine kernels), and replays on inputs changed in between give the
    bits of the workspace entry point."""
    lib = _capi.load()
    pb = make_problem(2, 4, 200, 1024, 128, seed=904, causal=True)
    splits = 3
    shape = (pb["B"], pb["H"], pb["Nq"], pb["D"])
    out = torch.full(shape, float("nan"), dtype=torch.float16, device=DEV)
    lse = torch.full(shape[:3], float("nan"), dtype=torch.float32, device=DEV)
    p = fill(pb, out, lse, splits)
    p.workspace, p.workspace_bytes = None, 0

    def call_static():
        rc = lib.intfa_fwd_full_int8_static(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, lib.intfa_error_string(rc)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                 # the first call on the device looks up the scratch array: outside the capture
        call_static()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call_static()
    g = torch.Generator(device=DEV).manual_seed(905)
    for rep in range(3):
        q = torch.randn(shape, generator=g, device=DEV, dtype=torch.float16)
        pb["t"][0].copy_((q * 40).round().clamp(-127, 127).to(torch.int8))      # new int8 Q, written by eager kernels
        out.fill_(float("nan")); lse.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        (o_ws, lse_ws), _ = run_both(pb, splits)
        assert torch.equal(out, o_ws) and torch.equal(lse, lse_ws), rep


def test_static_scratch_entry_point_rejects_what_does_not_fit():
    lib = _capi.load()
    pb = make_problem(1, 1, 8, 256, 128, seed=903, causal=False)
    out = torch.empty((1, 1, 8, 128), dtype=torch.float16, device=DEV)
    lse = torch.empty((1, 1, 8), dtype=torch.float32, device=DEV)
    p = fill(pb, out, lse, 2)
    # the same block described as a problem whose partials need 2 x 64 x 64 x 1024 x 129 x 4 bytes = 4 GiB: rejected before
    # anything is launched (the tensors are never touched)
    p.batch, p.heads, p.seqlen = 64, 64, 1024
    need = lib.intfa_fwd_workspace_bytes(ctypes.byref(p))
    assert need > _capi.STATIC_SCRATCH_BYTES
    rc = lib.intfa_fwd_full_int8_static(ctypes.byref(p), None)
    assert rc == -10 and b"INTFA_STATIC_SCRATCH_BYTES" in lib.intfa_error_string(rc)
    p.num_splits = 65
    assert lib.intfa_fwd_full_int8_static(ctypes.byref(p), None) == -8
    assert lib.intfa_fwd_full_int8_static(None, None) == -1
