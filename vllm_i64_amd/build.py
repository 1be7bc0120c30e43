"""Build the in-tree HIP libraries (gfx950 code objects + C ABI) with hipcc.  No GPU needed: hipcc cross-compiles.

libi64hip.so        the quantized token-routed-MoE forward (include/i64h.h)
libi64hip_dense.so  models with bf16 weights and a 32-bit residual: Linear, gated post-norm, latent attention, multi-stream
                    residual, state-space / gated recurrences, key-valued chunked attention, attention with separate keys and values,
                    gated linear recurrence, rotated attention with capped scores, gated delta rule, expert routing and grouped
                    expert Linears, sampling
                    (include/i64h_dense.h) - a library of its own, so that serving such a model builds nothing else
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libi64hip.so")
DENSE_OUT = os.path.join(HERE, "libi64hip_dense.so")
DENSE_SOURCES = ["i64h_api.hip", "i64h_dense.hip", "i64h_latent.hip", "i64h_hybrid.hip", "i64h_blocks.hip"]
SOURCES = ["i64h_api.hip", "i64h_route.hip", "i64h_quant.hip", "i64h_norm.hip", "i64h_gemm.hip", "i64h_gemm_os.hip", "i64h_attn.hip", "i64h_moe.hip", "i64h_fp8.hip", "i64h_kv.hip", "i64h_decode.hip", "i64h_variants.hip", "i64h_group_f32.hip", "i64h_lmhead.hip"]
# -ffp-contract=off: a*b+c stays two roundings unless the source says fmaf, so fp32 element-wise math has the
# same rounding steps as the reference's CPU ops.
# no packed-fp32 instructions: the compiler forms them from ordinary float code, and some of their forms have been unreliable
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-ffp-contract=off", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
         "-I", os.path.join(os.path.dirname(HERE), "include"), "-I", CSRC]


# per-file extras.  MFMA accumulators that element-wise code reads right after the matrix instructions (softmax on the
# scores, rescaling of the output tile) stay in ordinary VGPRs instead of being copied out of the accumulator registers.
EXTRA = {"i64h_attn.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}  # measured: no gain for the int8 GEMMs


def _stale(obj: str, src: str) -> bool:
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    # every object depends on both headers: the public one carries structs that cross translation units
    inc = os.path.join(os.path.dirname(HERE), "include")
    deps = [src, os.path.join(inc, "i64h.h"), os.path.join(inc, "i64h_dense.h"), os.path.abspath(__file__)]
    deps += [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    return any(os.path.getmtime(d) > t for d in deps)


def build(force: bool = False, verbose: bool = True, sources=None, out: str = OUT) -> str:
    sources = SOURCES if sources is None else sources
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    jobs = []
    for s in sources:
        src = os.path.join(CSRC, s)
        obj = os.path.join(objdir, s.replace(".hip", ".o"))
        if force or _stale(obj, src):
            jobs.append([hipcc, *FLAGS, *EXTRA.get(s, []), "-c", src, "-o", obj])

    def run(cmd):
        if verbose:
            print("[build]", os.path.basename(cmd[-3]), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed: {' '.join(cmd)}\n{r.stdout}\n{r.stderr}")
        # (the host pass does not know the device-only feature switch and says so once per function: not worth a line each)
        noise = [ln for ln in r.stderr.splitlines() if ln.strip() and "is not a recognized feature for this target" not in ln]
        if verbose and noise:
            print("\n".join(noise))

    with ThreadPoolExecutor(max_workers=min(6, max(1, len(jobs)))) as ex:
        list(ex.map(run, jobs))
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in sources]
    if jobs or not os.path.exists(out):
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", out]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    return out


def build_dense(force: bool = False, verbose: bool = True) -> str:
    return build(force=force, verbose=verbose, sources=DENSE_SOURCES, out=DENSE_OUT)


if __name__ == "__main__":
    if "--dense-only" not in sys.argv:
        print(build(force="--force" in sys.argv))
    print(build_dense(force="--force" in sys.argv))
