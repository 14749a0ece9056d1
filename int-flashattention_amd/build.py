"""Builds libintfa.so in-tree with hipcc for gfx950:  python -m int_flashattention_amd.build"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)
import spill_check  # noqa: E402  (a sibling module; this file also runs as a script)
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libintfa.so")
# -packed-fp32-ops is switched off on purpose: the compiler must not form v_pk_*_f32 from the float code.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


C_CALLER_SRC = os.path.join(os.path.dirname(HERE), "tests", "capi_c", "intfa_c_caller.c")
C_CALLER = C_CALLER_SRC[:-2]


def build_c_caller(verbose: bool = True) -> str:
    """Compiles the plain-C caller of the ABI (tests/capi_c) with gcc against include/intfa.h and libintfa.so."""
    root = os.path.dirname(HERE)
    cmd = ["gcc", "-std=c11", "-O2", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(root, "include"), "-I", "/opt/rocm/include",
           C_CALLER_SRC, "-o", C_CALLER, "-L", HERE, "-lintfa", "-L", "/opt/rocm/lib", "-lamdhip64", "-lm",
           "-Wl,-rpath,$ORIGIN/../../int-flashattention_amd", "-Wl,-rpath,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"gcc failed for {C_CALLER_SRC}:\n{r.stderr[-4000:]}")
    if verbose:
        print(f"built {C_CALLER}")
    return C_CALLER


RATE_PROBE_SRC = os.path.join(os.path.dirname(HERE), "bench_rate_probe.hip")
RATE_PROBE = RATE_PROBE_SRC[:-4]


def build_rate_probe(verbose: bool = True) -> str:
    """Compiles the stand-alone instruction-rate probe beside bench.py (measurement only; no library code in it)."""
    r = subprocess.run(["hipcc", *[f for f in FLAGS if f != "-fPIC"], RATE_PROBE_SRC, "-o", RATE_PROBE], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {RATE_PROBE_SRC}:\n{r.stderr[-4000:]}")
    if verbose:
        print(f"built {RATE_PROBE}")
    return RATE_PROBE


def build(verbose: bool = True, jobs: int = 8, only=None) -> str:
    """Compiles every source and links the library.  `only` (development): a list of name fragments - sources whose file
    name contains none of them keep their existing object file."""
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    srcs = sources()
    objs = [os.path.join(objdir, os.path.basename(s)[:-4] + ".o") for s in srcs]
    todo = [(s, o) for s, o in zip(srcs, objs)
            if not only or not os.path.exists(o) or any(frag in os.path.basename(s) for frag in only)]

    def compile_one(pair):
        # -save-temps=obj leaves the device assembly beside the object: it is scanned for register spills that lose lanes
        # (spill_check.py) and removed again with the other intermediate files
        src, obj = pair
        cmd = ["hipcc", *FLAGS, "-save-temps=obj", "-c", src, "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{r.stderr[-4000:]}")
        stem = os.path.basename(src)[:-4]
        findings, scanned = [], False
        for f in os.listdir(objdir):
            if not f.startswith(stem + "-") and not f.startswith(stem + ".hip-"):
                continue
            path = os.path.join(objdir, f)
            if f.endswith("gfx950.s"):
                with open(path) as fh:
                    findings = [f"{os.path.basename(src)}: {x}" for x in spill_check.scan(fh.read())]
                scanned = True
            os.remove(path)
        if not scanned:      # (a compiler that names its intermediate files otherwise must not pass unchecked)
            raise RuntimeError(f"no device assembly found for {src}: the spill scan did not run")
        return findings

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        findings = [x for fs in ex.map(compile_one, todo) for x in fs]
    if findings:
        raise RuntimeError("the compiler placed register spills where lanes are masked off (wrong results for those lanes):\n  "
                           + "\n  ".join(findings[:20]))
    r = subprocess.run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", OUT], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    if verbose:
        print(f"built {OUT} from {len(srcs)} source file(s), {len(todo)} compiled")
    if os.path.exists(C_CALLER_SRC):
        build_c_caller(verbose)
    if os.path.exists(RATE_PROBE_SRC) and not only:
        build_rate_probe(verbose)
    return OUT


if __name__ == "__main__":
    # python -m int_flashattention_amd.build [--only fragment,fragment,...]
    build(only=sys.argv[2].split(",") if len(sys.argv) > 2 and sys.argv[1] == "--only" else None)
    sys.exit(0)
