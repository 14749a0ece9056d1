"""Two host threads, each on a stream of its own, call the entry points at the same time: the library keeps no mutable
state between calls (the parameter block, the workspace and the stream are all the caller's), so every result must equal,
bit for bit, the result of the same call made alone.  Split-KV calls are in the mix: their partials live in a workspace
that the host wrapper allocates per call.  (The entry point with the static scratch buffer is excluded: calls to it that
overlap on one GPU race by contract.)
"""
import threading

import pytest
import torch

import intfa_oracle as O
import int_flashattention_amd as M

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _calls():
    g = torch.Generator().manual_seed(5)
    out = []
    for (B, H, Nq, Nk, D, causal, splits) in [(2, 4, 512, 512, 128, True, 1), (1, 8, 1, 4096, 128, False, 4), (2, 2, 300, 700, 64, False, 2),
                                               (1, 4, 384, 384, 256, True, 1)]:
        q = torch.randn((B, H, Nq, D), generator=g).half()
        k = torch.randn((B, H, Nk, D), generator=g).half()
        v = torch.randn((B, H, Nk, D), generator=g).half()
        q8, qs = O.quant_pertoken(q)
        k8, ks = O.quant_pertoken(k)
        v8, vs = O.quant_pertensor(v)
        sm = D ** -0.5
        t = [x.to(DEV) for x in (q, k, v, q8, qs, k8, ks, v8, vs)]
        q, k, v, q8, qs, k8, ks, v8, vs = t
        out.append(lambda q8=q8, k8=k8, v8=v8, qs=qs, ks=ks, vs=vs, c=causal, sm=sm, s=splits: M.attention_full_int8(q8, k8, v8, qs, ks, vs, c, sm, num_splits=s, p_round="rne"))
        out.append(lambda q8=q8, k8=k8, v=v, qs=qs, ks=ks, c=causal, sm=sm, s=splits: M.attention_int8(q8, k8, v, qs, ks, c, sm, num_splits=s))
        out.append(lambda q=q, k=k, v=v, c=causal, sm=sm, s=splits: M.attention(q, k, v, c, sm, num_splits=s))
    return out


def test_two_threads_on_two_streams_get_the_results_of_single_calls():
    calls = _calls()
    want = [f() for f in calls]
    torch.cuda.synchronize()
    errors = []

    def worker(order):
        try:
            stream = torch.cuda.Stream()                      # default priority
            with torch.cuda.stream(stream):
                for rep in range(6):
                    for i in order:
                        got = calls[i]()
                        stream.synchronize()
                        if not torch.equal(got, want[i]):
                            errors.append((rep, i))
        except Exception as e:                                  # surfaces in the main thread
            errors.append(repr(e))

    n = len(calls)
    a = threading.Thread(target=worker, args=(list(range(n)),))
    b = threading.Thread(target=worker, args=(list(reversed(range(n))),))
    a.start(); b.start(); a.join(); b.join()
    torch.cuda.synchronize()
    assert errors == []
