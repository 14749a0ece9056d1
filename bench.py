#!/usr/bin/env python3
"""Headline benchmark: full-int8 attention forward at B=4, H=32, N=4096, d=128 (non-causal) on one MI355X.

Prints ONE JSON line.  `value` is whole-job throughput in TOPS with the work model of the reference's harness,
ops = 4*B*H*N^2*d (x0.5 causal; benchmark.py:90-93), inputs resident in HBM before the timed region.
`roofline` prices the forward kernel against the dense int8 MFMA peak from per-launch HIP-event times;
`cpu_baseline` times the CPU oracle (a port of the reference's quantised arithmetic) on a bounded sample of the
same workload - one (batch, head) slice - on this box's host cores.
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
INT8_OPS_PER_CLK_CU = 8192   # v_mfma_i32_32x32x32_i8: 65536 ops in 8 passes of 4 clocks on each of a CU's 4 SIMDs
FP16_FLOPS_PER_CLK_CU = 4096


def device_peak_check(torch, dev):
    """The peak recomputed from what the device reports (compute units x maximum engine clock x ops per clock and CU: the
    first GPU agent of `rocminfo`, the compute-unit count also from the runtime), printed beside the datasheet constants
    the fractions are priced against."""
    import re
    import subprocess
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    name, mhz, cus_rocminfo = torch.cuda.get_device_properties(dev).name, None, None
    try:
        txt = subprocess.run(["/opt/rocm/bin/rocminfo"], capture_output=True, text=True, timeout=30).stdout
        for agent in txt.split("*******")[1:]:
            if re.search(r"Device Type:\s+GPU", agent):
                m = re.search(r"Max Clock Freq\. \(MHz\):\s+(\d+)", agent)
                c = re.search(r"Compute Unit:\s+(\d+)", agent)
                mhz = float(m.group(1)) if m else None
                cus_rocminfo = int(c.group(1)) if c else None
                break
    except Exception as e:          # rocminfo missing or unreadable: report what the runtime alone gives
        name += f" (rocminfo unavailable: {type(e).__name__})"
    out = {"device": name, "compute_units": cus, "compute_units_rocminfo": cus_rocminfo, "max_engine_clock_mhz": mhz,
           "int8_ops_per_clk_cu": INT8_OPS_PER_CLK_CU, "fp16_flops_per_clk_cu": FP16_FLOPS_PER_CLK_CU,
           "priced_against": {"int8_tops": INT8_PEAK_TOPS, "fp16_tflops": FP16_PEAK_TFLOPS, "hbm_gbs": HBM_PEAK_GBS}}
    if mhz:
        out["int8_tops"] = cus * mhz * 1e6 * INT8_OPS_PER_CLK_CU / 1e12
        out["fp16_tflops"] = cus * mhz * 1e6 * FP16_FLOPS_PER_CLK_CU / 1e12
    return out


# name: variant, B, H, N, D, causal, num_splits, input dtype, std of Q/K/V, fraction of K channels multiplied by 20
WORKLOADS = {
    "full_int8_B4_H32_N4096_d128": dict(variant="full", B=4, H=32, N=4096, D=128, causal=False, splits=1),
    "full_int8_B4_H32_N4096_d128_causal": dict(variant="full", B=4, H=32, N=4096, D=128, causal=True, splits=1),
    "half_int8_B8_H32_N2048_d128_causal": dict(variant="half", B=8, H=32, N=2048, D=128, causal=True, splits=1),
    "half_int8_B4_H32_N4096_d128": dict(variant="half", B=4, H=32, N=4096, D=128, causal=False, splits=1),
    "fp16_B4_H32_N4096_d128": dict(variant="fp", B=4, H=32, N=4096, D=128, causal=False, splits=1),
    # head_dim 256 of the two 16-bit-PV variants (eight-wave workgroups, two waves per 32 query rows)
    "half_int8_B4_H32_N4096_d256": dict(variant="half", B=4, H=32, N=4096, D=256, causal=False, splits=1),
    "fp16_B4_H32_N4096_d256": dict(variant="fp", B=4, H=32, N=4096, D=256, causal=False, splits=1),
    "full_int8_B1_H32_N16384_d128_causal_splitkv": dict(variant="full", B=1, H=32, N=16384, D=128, causal=True, splits=2,
                                                        k_outlier_frac=0.01),
    "full_int8_B1_H32_N16384_d128_causal": dict(variant="full", B=1, H=32, N=16384, D=128, causal=True, splits=1,
                                                k_outlier_frac=0.01),
    "full_int8_B16_H16_N1024_d64_bf16": dict(variant="full", B=16, H=16, N=1024, D=64, causal=False, splits=1,
                                             dtype="bfloat16", std=0.5),
    "full_int8_B16_H16_N1024_d256_bf16": dict(variant="full", B=16, H=16, N=1024, D=256, causal=False, splits=1,
                                              dtype="bfloat16", std=0.5),
    # the grid of the reference's own benchmark script (benchmark.py:23-45: BATCH, N_HEADS, HEAD_DIM = 4, 32, 64, N_CTX = 2^10 ..
    # 2^14, non-causal, providers full-int8 / int8 / fp16), with this build's input recipe
    "full_int8_B4_H32_N1024_d64": dict(variant="full", B=4, H=32, N=1024, D=64, causal=False, splits=1),
    "full_int8_B4_H32_N4096_d64": dict(variant="full", B=4, H=32, N=4096, D=64, causal=False, splits=1),
    "full_int8_B4_H32_N16384_d64": dict(variant="full", B=4, H=32, N=16384, D=64, causal=False, splits=1),
    "half_int8_B4_H32_N4096_d64": dict(variant="half", B=4, H=32, N=4096, D=64, causal=False, splits=1),
    "fp16_B4_H32_N4096_d64": dict(variant="fp", B=4, H=32, N=4096, D=64, causal=False, splits=1),
    "fp16_B4_H32_N4096_d64_causal": dict(variant="fp", B=4, H=32, N=4096, D=64, causal=True, splits=1),
    "half_int8_B4_H32_N4096_d64_causal": dict(variant="half", B=4, H=32, N=4096, D=64, causal=True, splits=1),
    # a number of (batch, head) pairs that is no multiple of the eight XCDs (how whole heads are pinned to one L2 then)
    "full_int8_B1_H12_N4096_d128": dict(variant="full", B=1, H=12, N=4096, D=128, causal=False, splits=1),
    # head_dim 256 at the headline's batch, heads and length (the eight-wave kernel of that head_dim)
    "full_int8_B4_H32_N4096_d256": dict(variant="full", B=4, H=32, N=4096, D=256, causal=False, splits=1),
    # the headline shape with V quantised per block of 128 keys and channel (the V scales of the reference's CUDA kernel)
    "full_int8_B4_H32_N4096_d128_vblock": dict(variant="full", B=4, H=32, N=4096, D=128, causal=False, splits=1, v_block=128),
    # the same with 64-key scale rows, the granularity of the reference's CUDA kernel (kBlockN = 64): two scale rows per key block
    "full_int8_B4_H32_N4096_d128_vblock64": dict(variant="full", B=4, H=32, N=4096, D=128, causal=False, splits=1, v_block=64),
    # decoding against a cache: one query per head, 16384 cached keys (HBM-bound: K and V are streamed once)
    "full_int8_decode_B8_H32_Nq1_Nk16384_d128": dict(variant="full", B=8, H=32, N=1, Nk=16384, D=128, causal=False, splits="auto"),
    "full_int8_decode_B32_H32_Nq1_Nk4096_d128": dict(variant="full", B=32, H=32, N=1, Nk=4096, D=128, causal=False, splits=1),
    "full_int8_decode_B32_H32_Nq1_Nk4096_d256": dict(variant="full", B=32, H=32, N=1, Nk=4096, D=256, causal=False, splits=1),
    # the same decode shape for the two variants with a 16-bit V cache (int8 or 16-bit K cache)
    "half_int8_decode_B32_H32_Nq1_Nk4096_d128": dict(variant="half", B=32, H=32, N=1, Nk=4096, D=128, causal=False, splits=1),
    "fp16_decode_B32_H32_Nq1_Nk4096_d128": dict(variant="fp", B=32, H=32, N=1, Nk=4096, D=128, causal=False, splits=1),
    "half_int8_decode_B32_H32_Nq1_Nk4096_d256": dict(variant="half", B=32, H=32, N=1, Nk=4096, D=256, causal=False, splits=1),
    "fp16_decode_B32_H32_Nq1_Nk4096_d256": dict(variant="fp", B=32, H=32, N=1, Nk=4096, D=256, causal=False, splits=1),
    # the input quantisers (HBM-bound): Q/K per token, V per (batch, head)
    "quant_pertoken_B4_H32_N4096_d128": dict(variant="quant_token", B=4, H=32, N=4096, D=128, causal=False, splits=1),
    "quant_pertensor_B4_H32_N4096_d128": dict(variant="quant_tensor", B=4, H=32, N=4096, D=128, causal=False, splits=1),
    "quant_perblock_channel_B4_H32_N4096_d128": dict(variant="quant_block", B=4, H=32, N=4096, D=128, causal=False, splits=1),
    # new keys and values of a whole prompt quantised into an empty int8 cache (the append of a prefill)
    "kvcache_append_B4_H32_N4096_d128": dict(variant="quant_append", B=4, H=32, N=4096, D=128, causal=False, splits=1),
}
# HBM bytes per launch of the forward kernel as measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE), each scaled by
# what the same counter reads for a plain copy of known size.  These are constants taken from the profile named beside
# them, NOT measured in the run that prints them (counters need the profiler); workloads without a profile report None.
MEASURED_TRAFFIC_BYTES = {
    # FETCH_SIZE x 1.9997 + WRITE_SIZE x 1.0 (KiB per dispatch, factors from a 256 MiB copy): 194.3 MiB read + 128 MiB written
    "full_int8_B4_H32_N4096_d128": (337941156, "profiles/fwd_full_int8_d128_B4_H32_N4096.txt"),
    # FETCH_SIZE x 1.9998 + WRITE_SIZE 256 x 1.0: 1032.2 MiB read + 0.25 MiB written (algorithmic: 1082523648)
    "full_int8_decode_B32_H32_Nq1_Nk4096_d128": (1082595402, "profiles/fwd_decode_full_int8_d128_B32_H32_Nq1_Nk4096.txt"),
}


def traffic_of(workload):
    t = MEASURED_TRAFFIC_BYTES.get(workload)
    return (t[0], f"constant from {t[1]} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured in this run)") if t else (None, None)


def ops_of(B, H, N, D, causal):
    return 4.0 * B * H * N * N * D * (0.5 if causal else 1.0)


def cpu_baseline(budget_s: float, w: dict):
    """The CPU oracle on a bounded sample of the timed workload: one (batch, head) slice of the same shape (same N, Nk, d,
    causal flag, variant and key-block length), for about `budget_s` seconds of CPU work.  The oracle is batched over
    (batch, head), so the rate of one slice is the rate of the whole workload on the same cores."""
    import torch
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import intfa_oracle as O
    cores = os.cpu_count() or 1
    cores = min(cores, 16) if os.environ.get("OMP_NUM_THREADS") is None else int(os.environ["OMP_NUM_THREADS"])
    torch.set_num_threads(cores)
    variant, N, D, causal = w["variant"], w["N"], w["D"], w["causal"]
    Nk = w.get("Nk", N)
    dt = getattr(torch, w.get("dtype", "float16"))
    g = torch.Generator().manual_seed(20)
    q = (torch.randn((1, 1, N, D), generator=g) * w.get("std", 1.0)).to(dt)
    k = (torch.randn((1, 1, Nk, D), generator=g) * w.get("std", 1.0)).to(dt)
    v = (torch.randn((1, 1, Nk, D), generator=g) * w.get("std", 1.0)).to(dt)
    sm = D ** -0.5
    if variant == "fp":
        fn = lambda: O.attention_fp(q, k, v, causal, sm, block_n=64)
    else:
        q8, qs = O.quant_pertoken(q); k8, ks = O.quant_pertoken(k)
        if variant == "full":
            bn = 128 if D == 128 else 64      # the kernels' key blocks (intfa_fwd_block_n)
            v_block = w.get("v_block")
            v8, vs = O.quant_perblock_channel(v, v_block) if v_block else O.quant_pertensor(v)
            kw = dict(v_scale_block=v_block) if v_block else {}
            fn = lambda: O.attention_full_int8(q8, k8, v8, qs, ks, vs, causal, sm, block_n=bn, out_dtype=dt, **kw)
        else:
            fn = lambda: O.attention_int8(q8, k8, v, qs, ks, causal, sm, block_n=64, out_dtype=dt)
    fn()
    times, t_end = [], time.perf_counter() + budget_s
    while len(times) < 3 or time.perf_counter() < t_end:
        t0 = time.perf_counter(); fn(); times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    ops = ops_of(1, 1, N, D, causal) * (Nk / N)
    return {"value": ops / med / 1e12, "unit": "TOPS", "cores": torch.get_num_threads(), "kind": "port", "ms": med * 1e3,
            "sample": f"1 of {w['B'] * w['H']} (batch, head) slices of the workload (N {N}, keys {Nk}, d {D}, "
                      f"{'causal' if causal else 'non-causal'}, {variant}), {len(times)} runs of the PyTorch CPU oracle, median"}


def bench_quant(args, variant, x, B, H, N, D, dt):
    """Times one quantiser; algorithmic bytes = 2 per element read + 1 written (+ scales); the per-(batch, head) variant
    reads its input twice (maximum, then quantise)."""
    import torch
    import int_flashattention_amd as M
    if variant == "quant_append":          # K and V of the prompt into an empty cache: reads both inputs once, writes both caches
        kc = torch.zeros((B, H, N, D), dtype=torch.int8, device=x.device); vc = torch.zeros_like(kc)
        ksc = torch.zeros((B, H, N), dtype=x.dtype, device=x.device)
        vs = (x.abs().amax(dim=(2, 3)) / 127).to(x.dtype)
        v_new = x.flip(2).contiguous()
        fn = lambda t: M.kvcache_append(kc, ksc, t, 0, vc, vs, v_new)
    else:
        fn = {"quant_token": M.quant_pertoken, "quant_tensor": M.quant_pertensor,
              "quant_block": lambda t: M.quant_perblock_channel(t, 128)}[variant]
    n = B * H * N * D
    # (the per-block variant reads its block twice too, but the second sweep of 32 KiB is served by the cache)
    scale_bytes = {"quant_token": 2 * B * H * N, "quant_tensor": 2 * B * H, "quant_block": 4 * B * H * (N // 128) * D,
                   "quant_append": 2 * B * H * N + 2 * B * H}[variant]
    alg_bytes = (2 + 1) * n * (2 if variant == "quant_append" else 1) + scale_bytes + (2 * n if variant == "quant_tensor" else 0)
    spin = device_spinup(torch, lambda: fn(x), args.spinup_ms)
    for _ in range(args.warmup):
        fn(x)
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for e0, e1 in evs:
        e0.record(); fn(x); e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per_launch_ms = [e0.elapsed_time(e1) for e0, e1 in evs]
    kern_ms = statistics.fmean(per_launch_ms)
    ms_step = wall * 1e3 / args.steps
    out = {"metric": "input quantiser throughput (algorithmic HBM bytes per second)", "value": alg_bytes / (ms_step * 1e-3) / 1e9,
           "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16->int8", "data": "synthetic",
           "config": {"workload": args.workload, "batch": B, "heads": H, "seqlen": N, "head_dim": D, "bytes_per_step": alg_bytes},
           "roofline": {"bound": "hbm", "achieved": alg_bytes / (kern_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": alg_bytes / (kern_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None,
                        "kernel": {"quant_token": "quant_pertoken_kernel", "quant_block": "quant_blockchan_kernel",
                                   "quant_tensor": "quant_slice_amax_kernel + quant_slice_apply_kernel",
                                   "quant_append": "kv_append_kernel (keys) + kv_append_kernel (values)"}[variant],
                        "avg_launch_ms": kern_ms, "median_launch_ms": statistics.median(per_launch_ms)},
           "peak_check": device_peak_check(torch, x.device), "device_spinup": spin}
    print(json.dumps(out))


def device_spinup(torch, step, ms):
    """The GPU's clock needs some tens of milliseconds of sustained load to leave its idle state: on these boxes the
    launch time of the headline kernel falls from 1.1 ms to its steady 0.85 ms over the first ~30 launches of a process,
    whatever ran before.  Five warm-up steps do not cover that, so the workload is run untimed for `ms` milliseconds
    first; the warm-up steps and the timed steps follow as the flags say."""
    if ms <= 0:
        return None
    t0 = time.perf_counter()
    n = 0
    first = last = None
    while (time.perf_counter() - t0) * 1e3 < ms:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(4):
            step()
        e1.record()
        torch.cuda.synchronize()
        last = e0.elapsed_time(e1) / 4
        first = last if first is None else first
        n += 4
    return {"ms": (time.perf_counter() - t0) * 1e3, "launches": n, "first_ms_per_launch": first, "last_ms_per_launch": last,
            "why": "untimed; lets the clock leave its idle state before the warm-up steps (launch times fall for ~30 ms after load begins)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--workload", default="full_int8_B4_H32_N4096_d128", choices=sorted(WORKLOADS))
    ap.add_argument("--p-round", default="reference", choices=["rne", "reference"])
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU-baseline budget; 0 skips it")
    ap.add_argument("--no-parity", action="store_true", help="skip the oracle check of one head")
    ap.add_argument("--no-other-rounding", action="store_true",
                    help="full-int8: do not also time the workload in the other rounding of P")
    ap.add_argument("--spinup-ms", type=float, default=80.0,
                    help="untimed: keep the GPU busy with the workload for this long before the warm-up steps, so that the "
                         "clock governor has left its idle state (0 = off); reported as device_spinup")
    ap.add_argument("--copy-probe-mib", type=int, default=0,
                    help="also run one device-to-device copy of this many MiB before the timed region: a kernel of known "
                         "HBM traffic that calibrates FETCH_SIZE / WRITE_SIZE when the run is under rocprofv3 --pmc")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (every (batch, head) is independent; there is no "
              "multi-GPU path to time). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    import int_flashattention_amd as M
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    w = WORKLOADS[args.workload]
    variant, B, H, N, D, causal, splits = w["variant"], w["B"], w["H"], w["N"], w["D"], w["causal"], w["splits"]
    dt = getattr(torch, w.get("dtype", "float16"))
    std = w.get("std", 1.0)
    sm = D ** -0.5
    g = torch.Generator(device=dev).manual_seed(20)
    Nk = w.get("Nk", N)
    mk = lambda n=N: (torch.randn((B, H, n, D), generator=g, device=dev, dtype=torch.float32) * std).to(dt)
    q, k, v = mk(), mk(Nk), mk(Nk)
    outlier_cols = []
    if w.get("k_outlier_frac"):
        n_out = max(1, round(w["k_outlier_frac"] * D))
        outlier_cols = torch.randperm(D, generator=torch.Generator().manual_seed(20))[:n_out].tolist()
        k[..., outlier_cols] = k[..., outlier_cols] * 20.0
    if variant.startswith("quant"):
        return bench_quant(args, variant, q, B, H, N, D, dt)
    bn = M.block_n(variant, D)
    if variant == "fp":
        step = lambda: M.attention(q, k, v, causal, sm, num_splits=splits)
    else:
        q8, qs = M.quant_pertoken(q)
        k8, ks = M.quant_pertoken(k)
        if variant == "full":
            v_block = w.get("v_block")
            v8, vs = M.quant_perblock_channel(v, v_block) if v_block else M.quant_pertensor(v)
            step = lambda: M.attention_full_int8(q8, k8, v8, qs, ks, vs, causal, sm, out_dtype=dt, num_splits=splits,
                                                 p_round=args.p_round, v_scale_block=v_block)
        else:
            step = lambda: M.attention_int8(q8, k8, v, qs, ks, causal, sm, num_splits=splits)
    ops = ops_of(B, H, N, D, causal) * (Nk / N)
    decode = Nk != N

    if args.copy_probe_mib > 0:
        src = torch.empty((args.copy_probe_mib << 20,), dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    spin = device_spinup(torch, step, args.spinup_ms)
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
    kern_med_ms = statistics.median(per_launch_ms)
    value = ops / (ms_step * 1e-3) / 1e12
    achieved = ops / (kern_ms * 1e-3) / 1e12

    # the same workload in the other rounding of P (full-int8 only), per-launch HIP events as above
    other_round = None
    if variant == "full" and not args.no_other_rounding:
        other = "reference" if args.p_round == "rne" else "rne"
        step_o = lambda: M.attention_full_int8(q8, k8, v8, qs, ks, vs, causal, sm, out_dtype=dt, num_splits=splits,
                                               p_round=other, v_scale_block=v_block)
        for _ in range(max(3, args.warmup // 5)):
            step_o()
        torch.cuda.synchronize()
        evo = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        for e0, e1 in evo:
            e0.record(); step_o(); e1.record()
        torch.cuda.synchronize()
        mo = [e0.elapsed_time(e1) for e0, e1 in evo]
        other_round = {"p_round": other, "avg_launch_ms": statistics.fmean(mo), "median_launch_ms": statistics.median(mo)}

    parity = None
    if not args.no_parity:
        # one (batch, head) slice of the timed problem against the CPU oracle run with the kernel's key-block length
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import intfa_oracle as O
        o = step(); torch.cuda.synchronize()
        b, h = B - 1, H - 1
        c = lambda t: t[b:b + 1, h:h + 1].cpu()
        got = o[b:b + 1, h:h + 1].float().cpu()
        exact = O.attention_exact(c(q), c(k), c(v), causal, sm).float()
        refs = {}
        if variant == "full":
            a8 = (c(q8), c(k8), c(v8), c(qs), c(ks), c(vs), causal, sm)
            okw = dict(v_scale_block=v_block) if v_block else {}
            if splits != "auto" and splits > 1:
                # a split restarts the running maximum, so its P8 is quantised in another frame than the single pass:
                # the oracle evaluated with the same split is the reference; the single pass is shown beside it
                refs["vs_oracle_split_reference_rounding"] = O.attention_full_int8_splitkv(*a8, splits, block_n=bn, out_dtype=dt)
                refs["vs_single_pass_reference_rounding"] = O.attention_full_int8(*a8, block_n=bn, out_dtype=dt)
            else:
                refs["vs_reference_rounding"] = O.attention_full_int8(*a8, block_n=bn, out_dtype=dt, **okw)
            if splits == "auto":
                refs = {"vs_single_pass_reference_rounding": O.attention_full_int8(*a8, block_n=bn, out_dtype=dt, **okw)}
            if args.p_round == "rne" and splits == 1:
                refs["vs_same_rounding"] = O.attention_full_int8(*a8, block_n=bn, out_dtype=dt, p_requant=O.p_requant_rne, **okw)
        elif variant == "half":
            refs["vs_oracle"] = O.attention_int8(c(q8), c(k8), c(v), c(qs), c(ks), causal, sm, block_n=bn, out_dtype=dt)
        else:
            refs["vs_oracle"] = O.attention_fp(c(q), c(k), c(v), causal, sm, block_n=bn)
        # max_abs / mean_rel (= mean|x-y| / mean|y|) are the measures the tolerances are stated in; mre_reference is the
        # reference harness's own measure (benchmark.py:110-122: mean(|y-x| / (|y| + 1e-5)), x the kernel's output), over
        # every element of the slice and over the last four (its CALC_NUM = 4)
        err = lambda x, y: {"max_abs": (x - y).abs().max().item(), "mean_rel": ((x - y).abs().mean() / y.abs().mean()).item(),
                            "mre_reference": O.mean_relative_error(x, y),
                            "mre_reference_calc_num_4": O.mean_relative_error(x, y, calc_num=4)}
        parity = {"slice": f"batch {b}, head {h}", "oracle_block_n": bn}
        for name, r in refs.items():
            parity[name] = err(got, r.float())
        parity["vs_exact_attention"] = err(got, exact)
        first = next(iter(refs.values())).float()
        parity["oracle_vs_exact_attention"] = err(first, exact)

    if variant == "full":
        peak, peak_model, dtype_s = INT8_PEAK_TOPS, "256 CU x 2.4 GHz x 8192 int8 ops/clk/CU", "int8"
    elif variant == "half":
        peak = 1.0 / (0.5 / INT8_PEAK_TOPS + 0.5 / FP16_PEAK_TFLOPS)
        peak_model, dtype_s = "half of the ops at the int8 rate (5033 T), half at the fp16 rate (2517 T)", "int8+f16"
    else:
        peak, peak_model, dtype_s = FP16_PEAK_TFLOPS, "256 CU x 2.4 GHz x 4096 fp16 flops/clk/CU", "f16"
    kernel_name = "fwd_full_int8_kernel" if variant == "full" else "fwd_f16pv_kernel"
    out = {
        "metric": "attention fwd TOPS + % int8 MFMA peak, B4 H32 N4096 d128 full-int8",
        "value": value, "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype_s, "data": "synthetic",
        "config": {"workload": args.workload, "variant": variant, "batch": B, "heads": H, "seqlen": N, "head_dim": D,
                   "causal": causal, "num_splits": splits, "p_round": args.p_round, "ops_per_step": ops,
                   "key_block": bn, "io_dtype": str(dt).replace("torch.", ""),
                   "inputs": f"Q,K,V {str(dt).replace('torch.', '')} ~ N(0,{std}), seed 20"
                             + (f", K channels {outlier_cols} x20" if outlier_cols else "")
                             + ("; Q,K per-token int8" if variant != "fp" else "")
                             + ((f", V int8 per block of {w['v_block']} keys and channel" if w.get("v_block")
                                 else ", V per-(batch,head) int8") if variant == "full" else "")},
        "pct_int8_peak": 100.0 * value / INT8_PEAK_TOPS,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": peak, "unit": "TOP/s" if variant == "full" else "TFLOP/s",
                     "frac": achieved / peak, "traffic": traffic_of(args.workload)[0], "traffic_source": traffic_of(args.workload)[1],
                     "kernel": kernel_name, "avg_launch_ms": kern_ms, "median_launch_ms": kern_med_ms,
                     "achieved_at_median": ops / (kern_med_ms * 1e-3) / 1e12, "peak_model": peak_model,
                     "launch_includes": "forward kernel" + (" + split-KV combine kernel" if splits != 1 else "")},
        "peak_check": device_peak_check(torch, dev),
        "device_spinup": spin,
    }
    if other_round is not None:
        a_o = ops / (other_round["avg_launch_ms"] * 1e-3) / 1e12
        out["roofline_" + other_round["p_round"] + "_rounding"] = {
            "bound": "mfma", "achieved": a_o, "peak": peak, "unit": "TOP/s", "frac": a_o / peak, "kernel": kernel_name,
            "p_round": other_round["p_round"], "avg_launch_ms": other_round["avg_launch_ms"],
            "median_launch_ms": other_round["median_launch_ms"],
            "slowdown_vs_timed_rounding": other_round["avg_launch_ms"] / kern_ms}
    if decode:
        # one pass over the cached K and V and the k scales; Q, O and the split partials are a rounding error
        sb = 2 if dt != torch.float32 else 4
        k_bytes = 1 if variant in ("full", "half") else 2
        v_bytes = 1 if variant == "full" else 2
        alg_bytes = B * H * Nk * (D * (k_bytes + v_bytes) + (sb if variant != "fp" else 0)) + B * H * N * D * (k_bytes + 2)
        gbs = alg_bytes / (kern_ms * 1e-3) / 1e9
        vname = {"full": "full-int8", "half": "half-int8", "fp": "fp16"}[variant]
        out["metric"] = f"decode attention: cached K+V bytes streamed per second ({vname}, one query per head)"
        out["value"], out["unit"] = alg_bytes / (ms_step * 1e-3) / 1e9, "GB/s"
        out["config"]["seqlen_k"] = Nk
        out["config"]["bytes_per_step"] = alg_bytes
        out.pop("pct_int8_peak")
        out["roofline"] = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                           "traffic": traffic_of(args.workload)[0], "traffic_source": traffic_of(args.workload)[1],
                           "kernel": "fwd_decode_full_int8_kernel" if variant == "full" else "fwd_decode_f16pv_kernel", "avg_launch_ms": kern_ms, "median_launch_ms": kern_med_ms,
                           "launch_includes": "forward kernel" + (" + split-KV combine kernel" if splits != 1 else "")}
        if other_round is not None:         # the same bytes over the other rounding's launch time
            g_o = alg_bytes / (other_round["avg_launch_ms"] * 1e-3) / 1e9
            out["roofline_" + other_round["p_round"] + "_rounding"].update(
                {"bound": "hbm", "achieved": g_o, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": g_o / HBM_PEAK_GBS,
                 "kernel": out["roofline"]["kernel"]})
    if parity is not None:
        out["parity"] = parity
    if args.cpu_seconds > 0:
        out["cpu_baseline"] = cpu_baseline(args.cpu_seconds, w)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
