"""CPU-side checks of the drop-in boundary: the C ABI library loads and exports what include/intfa.h
declares, the ctypes mirror of the parameter block has the C layout, argument validation rejects bad
blocks before any GPU call, and the Python entry points keep the reference's checks."""
import ctypes
import os
import re
import subprocess
import tempfile

import pytest
import torch

import int_flashattention_amd as M
from int_flashattention_amd import _capi, _host

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "intfa.h")


def test_library_exports_every_declared_symbol():
    lib = _capi.load()
    text = open(HEADER).read()
    declared = sorted(set(re.findall(r"^\s*(?:int|size_t|const char\*)\s+(intfa_\w+)\s*\(", text, flags=re.M)))
    assert declared, "no declarations parsed from include/intfa.h"
    assert set(declared) == set(_capi.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in intfa.h but not exported by libintfa.so"
    header_version = int(re.search(r"#define INTFA_VERSION (\d+)", text).group(1))
    assert lib.intfa_version() == header_version == _capi.ABI_VERSION
    assert lib.intfa_fwd_block_n(0, 128) == 128 == _host.BLOCK
    assert lib.intfa_fwd_block_n(0, 64) == 64      # never longer than head_dim (flash_atten_full_int8.py:88)
    assert lib.intfa_fwd_block_n(0, 256) == 64 and lib.intfa_fwd_block_n(1, 128) == 64 and lib.intfa_fwd_block_n(2, 64) == 64
    assert lib.intfa_fwd_block_n(3, 128) < 0 and lib.intfa_fwd_block_n(0, 96) < 0


def test_ctypes_struct_matches_c_layout():
    """Compiles a tiny C program against include/intfa.h and compares sizeof/offsetof with the ctypes mirror."""
    fields = [f[0] for f in _capi.FwdParams._fields_]
    body = "".join(f'printf("{f} %zu\\n", offsetof(intfa_fwd_params, {f}));\n' for f in fields)
    src = f'#include <stdio.h>\n#include <stddef.h>\n#include "intfa.h"\nint main(void){{\n{body}printf("sizeof %zu\\n", sizeof(intfa_fwd_params));return 0;}}\n'
    with tempfile.TemporaryDirectory() as td:
        c = os.path.join(td, "layout.c"); exe = os.path.join(td, "layout")
        open(c, "w").write(src)
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), c, "-o", exe], check=True)
        out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout
    got = dict(line.split() for line in out.strip().splitlines())
    for f in fields:
        assert int(got[f]) == getattr(_capi.FwdParams, f).offset, f
    assert int(got["sizeof"]) == ctypes.sizeof(_capi.FwdParams)


def test_append_struct_matches_c_layout():
    fields = [f[0] for f in _capi.AppendParams._fields_]
    body = "".join(f'printf("{f} %zu\\n", offsetof(intfa_append_params, {f}));\n' for f in fields)
    src = f'#include <stdio.h>\n#include <stddef.h>\n#include "intfa.h"\nint main(void){{\n{body}printf("sizeof %zu\\n", sizeof(intfa_append_params));return 0;}}\n'
    with tempfile.TemporaryDirectory() as td:
        c = os.path.join(td, "layout.c"); exe = os.path.join(td, "layout")
        open(c, "w").write(src)
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), c, "-o", exe], check=True)
        out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout
    got = dict(line.split() for line in out.strip().splitlines())
    for f in fields:
        assert int(got[f]) == getattr(_capi.AppendParams, f).offset, f
    assert int(got["sizeof"]) == ctypes.sizeof(_capi.AppendParams)


def test_append_validation_rejects_bad_blocks_before_touching_the_gpu():
    lib = _capi.load()

    def block(**kw):
        a = _capi.AppendParams()
        for n in ("k_new", "v_new", "k_cache", "v_cache", "k_scale_cache", "v_scale", "seqlens_k"):
            setattr(a, n, 0x10000)
        a.batch, a.heads_kv, a.seqlen_new, a.seqlen_cache, a.head_dim, a.dtype = 2, 3, 4, 64, 32, _capi.INTFA_F16
        for t in ("kn", "vn"):
            setattr(a, f"{t}_stride_b", 3 * 4 * 32); setattr(a, f"{t}_stride_h", 4 * 32); setattr(a, f"{t}_stride_n", 32)
        for t in ("kc", "vc"):
            setattr(a, f"{t}_stride_b", 3 * 64 * 32); setattr(a, f"{t}_stride_h", 64 * 32); setattr(a, f"{t}_stride_n", 32)
        a.ksc_stride_b, a.ksc_stride_h, a.ksc_stride_n = 3 * 64, 64, 1
        a.vs_stride_b, a.vs_stride_h = 3, 1
        for k, v in kw.items():
            setattr(a, k, v)
        return a
    rc = lambda **kw: lib.intfa_kvcache_append_int8(ctypes.byref(block(**kw)), None)
    assert lib.intfa_kvcache_append_int8(None, None) == -1
    assert rc(k_new=None) == -1 and rc(k_cache=None) == -1 and rc(k_scale_cache=None) == -1
    assert rc(v_cache=None) == -1 and rc(v_scale=None) == -1            # v_new given: its cache and scale are required
    assert rc(batch=0) == -7 and rc(heads_kv=0) == -7
    assert rc(seqlen_new=0) == -3 and rc(seqlen_cache=0) == -3
    assert rc(seqlens_k=None, seqlen_filled=65) == -3 and rc(seqlens_k=None, seqlen_filled=-1) == -3
    assert rc(head_dim=48) == -2 and rc(dtype=_capi.INTFA_F32) == -5
    assert rc(k_new=0x10008) == -4 and rc(kn_stride_n=36) == -4 and rc(k_cache=0x10004) == -4 and rc(vc_stride_h=12) == -4
    assert rc(seqlens_k=0x10002) == -4
    assert rc(kn_stride_n=16) == -7 and rc(vc_stride_n=16) == -7


def _valid_block():
    """A parameter block that passes validation (pointers are fake but aligned; it is never launched)."""
    p = _capi.FwdParams()
    for n in ("q", "k", "v", "out", "q_scale", "k_scale", "v_scale"):
        setattr(p, n, 0x10000)
    p.batch, p.heads, p.seqlen, p.head_dim = 1, 2, 256, 128
    for t in ("q", "k", "v", "o"):
        setattr(p, f"{t}_stride_b", 2 * 256 * 128); setattr(p, f"{t}_stride_h", 256 * 128); setattr(p, f"{t}_stride_n", 128)
    p.qs_stride_b, p.qs_stride_h, p.qs_stride_n = 512, 256, 1
    p.ks_stride_b, p.ks_stride_h, p.ks_stride_n = 512, 256, 1
    p.vs_stride_b, p.vs_stride_h = 2, 1
    p.sm_scale = 0.1
    return p


@pytest.mark.parametrize("mutate, code", [
    (lambda p: setattr(p, "q", None), -1),
    (lambda p: setattr(p, "v_scale", None), -1),
    (lambda p: setattr(p, "head_dim", 48), -2),
    (lambda p: setattr(p, "seqlen", -128), -3),
    (lambda p: setattr(p, "seqlen", 0), -3),
    (lambda p: setattr(p, "k", 0x10008), -4),
    (lambda p: setattr(p, "q_stride_n", 120), -4),
    (lambda p: setattr(p, "out", 0x10008), -4),            # the output rows are stored 16 bytes per lane
    (lambda p: setattr(p, "o_stride_n", 132), -4),         # 264 bytes: a multiple of 8 only
    (lambda p: setattr(p, "scale_dtype", 7), -5),
    (lambda p: setattr(p, "io_dtype", 2), -5),
    (lambda p: setattr(p, "num_splits", 4), -6),          # splits requested without a workspace
    (lambda p: setattr(p, "batch", 0), -7),
    (lambda p: setattr(p, "heads_kv", 3), -7),             # K/V heads must divide the query heads
    (lambda p: setattr(p, "q_stride_n", 64), -7),          # rows overlap: stride below head_dim
    (lambda p: (setattr(p, "seqlen", 1 << 20), setattr(p, "k_stride_n", 1 << 13)), -7),   # a K slice of 8 GiB
    (lambda p: (setattr(p, "num_splits", 65), setattr(p, "workspace", 0x10000), setattr(p, "workspace_bytes", 1 << 40)), -8),
    (lambda p: (setattr(p, "v_scale_block", 32), setattr(p, "vs_stride_blk", 128)), -9),    # neither a multiple of the key block (128) nor 64
    (lambda p: (setattr(p, "v_scale_block", 192), setattr(p, "vs_stride_blk", 128)), -9),   # a multiple of 64 only
    (lambda p: (setattr(p, "v_scale_block", 128), setattr(p, "vs_stride_blk", 64)), -9),    # scale rows overlap
    (lambda p: setattr(p, "v_scale_block", -1), -9),
    (lambda p: setattr(p, "seqlen_k", -5), -3),
    (lambda p: setattr(p, "causal_rows", 4), -3),                                            # only with causal
    (lambda p: (setattr(p, "causal", 1), setattr(p, "causal_rows", 4)), -3),                # 256 rows: not a decode shape
    (lambda p: (setattr(p, "causal", 1), setattr(p, "seqlen", 48), setattr(p, "causal_rows", 5)), -3),   # 48 % 5 != 0
    (lambda p: setattr(p, "seqlens_k", 0x10002), -4),
    (lambda p: (setattr(p, "v_scale_block", 128), setattr(p, "vs_stride_blk", 128), setattr(p, "v_scale", 0x10002)), -4),
])
def test_validation_rejects_bad_blocks_before_touching_the_gpu(mutate, code):
    lib = _capi.load()
    p = _valid_block()
    mutate(p)
    assert lib.intfa_fwd_full_int8(ctypes.byref(p), None) == code
    assert lib.intfa_error_string(code).decode() not in ("", "ok")


def test_null_block_and_error_strings():
    lib = _capi.load()
    assert lib.intfa_fwd_full_int8(None, None) == -1
    assert lib.intfa_fwd_half_int8(None, None) == -1
    assert lib.intfa_fwd_fp16(None, None) == -1
    assert lib.intfa_error_string(0) == b"ok"
    assert lib.intfa_error_string(700) == b"hip error"


def test_workspace_query():
    lib = _capi.load()
    p = _valid_block()
    assert lib.intfa_fwd_workspace_bytes(ctypes.byref(p)) == 0
    p.num_splits = 4
    rows = 4 * 1 * 2 * 256
    assert lib.intfa_fwd_workspace_bytes(ctypes.byref(p)) == rows * 128 * 4 + rows * 4


def test_entry_points_keep_the_reference_asserts():
    q = torch.zeros((1, 1, 128, 48), dtype=torch.int8)
    s = torch.ones((1, 1, 128), dtype=torch.float16)
    with pytest.raises(AssertionError):                    # head dim not in {16, 32, 64, 128, 256}
        _host.check_head_dims(q, q, q)
    with pytest.raises(AssertionError):                    # q/k/v head dims differ
        _host.check_head_dims(torch.zeros((1, 1, 128, 64)), torch.zeros((1, 1, 128, 32)), torch.zeros((1, 1, 128, 64)))
    q = torch.zeros((1, 1, 128, 64), dtype=torch.int8)
    with pytest.raises(RuntimeError, match="GPU only"):     # no CPU fallback
        M.attention_full_int8(q, q, q, s, s, torch.ones((1, 1), dtype=torch.float16), False, 1.0, p_round="rne")


def test_split_count_heuristic():
    lib = _capi.load()
    p = _capi.FwdParams()
    p.batch, p.heads, p.seqlen, p.head_dim = 4, 32, 4096, 128
    assert lib.intfa_fwd_suggest_splits(ctypes.byref(p), 0, 256) == 1              # 4096 workgroups fill 256 CUs
    p.batch, p.heads, p.seqlen, p.seqlen_k = 1, 8, 1, 8192                          # decoding: 8 workgroups
    assert lib.intfa_fwd_suggest_splits(ctypes.byref(p), 0, 256) == 16             # 64 key blocks, four per split
    assert lib.intfa_fwd_suggest_splits(ctypes.byref(p), 1, 256) == 32             # 64-key blocks: 128 of them
    assert lib.intfa_fwd_suggest_splits(ctypes.byref(p), 0, 0) == 16               # default device size
    p.batch, p.heads, p.seqlen_k = 2, 64, 4096                                      # 128 decode workgroups
    assert lib.intfa_fwd_suggest_splits(ctypes.byref(p), 1, 256) == 4              # head_dim 128: two workgroups per CU
    p.head_dim = 256
    assert lib.intfa_fwd_suggest_splits(ctypes.byref(p), 1, 256) == 2              # head_dim 256: one per CU
    p.batch, p.heads, p.head_dim = 1, 8, 128
    p.seqlen_k = 256
    assert lib.intfa_fwd_suggest_splits(ctypes.byref(p), 0, 256) == 1              # too few key blocks to split
    p.batch, p.heads, p.seqlen, p.seqlen_k = 1, 32, 1024, 0
    assert lib.intfa_fwd_suggest_splits(ctypes.byref(p), 0, 256) == 2              # 256 workgroups on 512 slots
    assert lib.intfa_fwd_suggest_splits(ctypes.byref(p), 7, 256) == -5 and lib.intfa_fwd_suggest_splits(None, 0, 256) == -1
    p.head_dim = 100
    assert lib.intfa_fwd_suggest_splits(ctypes.byref(p), 0, 256) == -2


def test_quantisers_refuse_cpu_tensors_and_bad_arguments():
    x = torch.randn((2, 3, 16, 32)).half()
    for fn in (M.quant_pertoken, M.quant_pertensor):
        with pytest.raises(RuntimeError, match="GPU only"):     # no CPU fallback
            fn(x)
    lib = _capi.load()
    one = ctypes.c_void_p(16)            # a non-null, 16-byte aligned address: validation happens before any launch
    ok = dict(x=one, sb=96 * 32, sh=32 * 32, sn=32, q8=one, scale=one, B=2, H=3, N=32, d=32, dt=_capi.INTFA_F16)

    def call(**kw):
        a = dict(ok, **kw)
        return lib.intfa_quant_pertoken(a["x"], a["sb"], a["sh"], a["sn"], a["q8"], a["scale"], a["B"], a["H"], a["N"], a["d"],
                                        a["dt"], None)
    assert call(x=None) == -1 and call(q8=None) == -1 and call(scale=None) == -1
    assert call(d=48) == -2 and call(dt=_capi.INTFA_F32) == -5 and call(B=0) == -7
    assert call(sn=33) == -4 and call(x=ctypes.c_void_p(8)) == -4
    assert call(sn=24) == -7 and call(sn=16, d=32) == -7        # rows shorter than head_dim would overlap
    assert lib.intfa_quant_pertensor_workspace_bytes(4, 32) == 4 * 32 * 4
    rc = lib.intfa_quant_pertensor(one, 96 * 32, 32 * 32, 32, one, one, 2, 3, 32, 32, _capi.INTFA_F16, None, 0, None)
    assert rc == -6
