#!/usr/bin/env python3
"""Headline benchmark: full-int8 attention forward at B=4, H=32, N=4096, d=128 (non-causal) on one MI355X.

Prints ONE JSON line.  `value` is whole-job throughput in TOPS with the work model of the reference's harness,
ops = 4*B*H*N^2*d (x0.5 causal; benchmark.py:90-93), inputs resident in HBM before the timed region.
`roofline` prices the forward kernel against the dense int8 MFMA peak from per-launch HIP-event times;
`cpu_baseline` times the CPU oracle (a port of the reference's quantised arithmetic) on the benchmark's
CPU-runnable configuration on this box's host cores.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

INT8_PEAK_TOPS = 5033.0      # MI355X dense int8 MFMA: 256 CUs x 2.4 GHz x 8192 ops/clk/CU
FP16_PEAK_TFLOPS = 2516.6
HBM_PEAK_GBS = 8000.0

WORKLOADS = {
    # name: (variant, B, H, N, D, causal, splits)
    "full_int8_B4_H32_N4096_d128": ("full", 4, 32, 4096, 128, False, 1),
    "full_int8_B4_H32_N4096_d128_causal": ("full", 4, 32, 4096, 128, True, 1),
    "half_int8_B8_H32_N2048_d128_causal": ("half", 8, 32, 2048, 128, True, 1),
    "full_int8_B1_H32_N16384_d128_causal_splitkv": ("full", 1, 32, 16384, 128, True, 2),
    "full_int8_B16_H16_N1024_d64": ("full", 16, 16, 1024, 64, False, 1),
    "full_int8_B16_H16_N1024_d256": ("full", 16, 16, 1024, 256, False, 1),
}


def ops_of(B, H, N, D, causal):
    return 4.0 * B * H * N * N * D * (0.5 if causal else 1.0)


def cpu_baseline(budget_s: float):
    """The CPU oracle on B=1, H=4, N=256, d=64, non-causal, for about `budget_s` seconds of CPU work."""
    import torch
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import intfa_oracle as O
    cores = os.cpu_count() or 1
    cores = min(cores, 16) if os.environ.get("OMP_NUM_THREADS") is None else int(os.environ["OMP_NUM_THREADS"])
    torch.set_num_threads(cores)
    B, H, N, D = 1, 4, 256, 64
    q, k, v, _ = O.make_inputs(B, H, N, D, seed=20)
    q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k); v8, vs = O.quant_pertensor(v)
    fn = lambda: O.attention_full_int8(q8, k8, v8, qs, ks, vs, False, D ** -0.5, block_n=128)
    for _ in range(3):
        fn()
    times, t_end = [], time.perf_counter() + budget_s
    while len(times) < 10 or time.perf_counter() < t_end:
        t0 = time.perf_counter(); fn(); times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    return {"value": ops_of(B, H, N, D, False) / med / 1e12, "unit": "TOPS", "cores": torch.get_num_threads(),
            "kind": "port", "ms": med * 1e3,
            "sample": f"{len(times)} runs of the PyTorch CPU oracle, full-int8 B{B} H{H} N{N} d{D} non-causal, median"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--workload", default="full_int8_B4_H32_N4096_d128", choices=sorted(WORKLOADS))
    ap.add_argument("--p-round", default="rne", choices=["rne", "reference"])
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU-baseline budget; 0 skips it")
    ap.add_argument("--no-parity", action="store_true", help="skip the oracle check of one head")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (every (batch, head) is independent; there is no "
              "multi-GPU path to time). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    import int_flashattention_amd as M
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    variant, B, H, N, D, causal, splits = WORKLOADS[args.workload]
    sm = D ** -0.5
    g = torch.Generator(device=dev).manual_seed(20)
    dt = torch.float16
    q = torch.randn((B, H, N, D), generator=g, device=dev, dtype=dt)
    k = torch.randn((B, H, N, D), generator=g, device=dev, dtype=dt)
    v = torch.randn((B, H, N, D), generator=g, device=dev, dtype=dt)
    q8, qs = M.quant_pertoken(q)
    k8, ks = M.quant_pertoken(k)
    if variant == "full":
        v8, vs = M.quant_pertensor(v)
        step = lambda: M.attention_full_int8(q8, k8, v8, qs, ks, vs, causal, sm, num_splits=splits, p_round=args.p_round)
    elif variant == "half":
        step = lambda: M.attention_int8(q8, k8, v, qs, ks, causal, sm, num_splits=splits)
    else:
        step = lambda: M.attention(q, k, v, causal, sm, num_splits=splits)
    fp_slice = tuple(t[B - 1:B, H - 1:H].cpu() for t in (q, k, v))
    del q, k
    ops = ops_of(B, H, N, D, causal)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # per-launch device times: HIP events on the stream the kernels are launched on (torch's current stream)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for e0, e1 in evs:
        e0.record(); step(); e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per_launch_ms = [e0.elapsed_time(e1) for e0, e1 in evs]
    ms_step = wall * 1e3 / args.steps
    kern_ms = statistics.fmean(per_launch_ms)
    value = ops / (ms_step * 1e-3) / 1e12
    achieved = ops / (kern_ms * 1e-3) / 1e12

    parity = None
    if not args.no_parity and variant == "full":
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import intfa_oracle as O
        o = step(); torch.cuda.synchronize()
        b, h, rows = B - 1, H - 1, min(N, 4096)
        c = lambda t: t[b:b + 1, h:h + 1].cpu()
        rq = O.p_requant_rne if args.p_round == "rne" else O.p_requant_reference
        if splits > 1:
            ref_same = O.attention_full_int8_splitkv(c(q8), c(k8), c(v8), c(qs), c(ks), c(vs), causal, sm, splits, block_n=128)
            ref = ref_same
        else:
            ref_same = O.attention_full_int8(c(q8), c(k8), c(v8), c(qs), c(ks), c(vs), causal, sm, block_n=128, p_requant=rq)
            ref = O.attention_full_int8(c(q8), c(k8), c(v8), c(qs), c(ks), c(vs), causal, sm, block_n=128)
        got = o[b:b + 1, h:h + 1].float().cpu()
        exact = O.attention_exact(*fp_slice, causal, sm).float()
        d1 = (got - ref.float()).abs(); d2 = (got - ref_same.float()).abs(); d3 = (got - exact).abs()
        d4 = (ref.float() - exact).abs()
        parity = {"slice": f"batch {b}, head {h}",
                  "vs_reference_rounding": {"max_abs": d1.max().item(), "mean_rel": (d1.mean() / ref.float().abs().mean()).item()},
                  "vs_same_rounding": {"max_abs": d2.max().item(), "mean_rel": (d2.mean() / ref_same.float().abs().mean()).item()},
                  "vs_exact_fp16_attention": {"max_abs": d3.max().item(), "mean_rel": (d3.mean() / exact.abs().mean()).item()},
                  "oracle_vs_exact_fp16_attention": {"max_abs": d4.max().item(), "mean_rel": (d4.mean() / exact.abs().mean()).item()}}

    out = {
        "metric": "attention fwd TOPS + % int8 MFMA peak, B4 H32 N4096 d128 full-int8",
        "value": value, "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8" if variant == "full" else ("int8+f16" if variant == "half" else "f16"),
        "data": "synthetic",
        "config": {"workload": args.workload, "variant": variant, "batch": B, "heads": H, "seqlen": N, "head_dim": D,
                   "causal": causal, "num_splits": splits, "p_round": args.p_round, "ops_per_step": ops,
                   "inputs": "Q,K,V fp16 ~ N(0,1), seed 20; Q,K per-token int8, V per-(batch,head) int8"},
        "pct_int8_peak": 100.0 * value / INT8_PEAK_TOPS,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                     "frac": achieved / INT8_PEAK_TOPS, "traffic": None,
                     "kernel": "fwd_int8_kernel", "avg_launch_ms": kern_ms,
                     "peak_model": "256 CU x 2.4 GHz x 8192 int8 ops/clk/CU"},
    }
    if parity is not None:
        out["parity"] = parity
    if args.cpu_seconds > 0:
        out["cpu_baseline"] = cpu_baseline(args.cpu_seconds)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
