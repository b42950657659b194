"""Builds libflashstu_hip.so for gfx950 with hipcc (no GPU needed)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["fstu_core.hip", "fstu_linear.hip", "fstu_stu.hip", "fstu_fft.hip", "fstu_attn.hip", "fstu_attn_mfma.hip", "fstu_pack.hip", "fstu_mlp.hip", "fstu_lds_seq.hip", "fstu_gemm.hip", "fstu_gemm_any.hip", "fstu_engine.hip"]
LIB = os.path.join(HERE, "libflashstu_hip.so")
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
         # packed fp32 instructions are kept out of the generated code
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# The first 16 kernel-argument dwords are preloaded into SGPRs by the command processor instead of being fetched by
# the kernel's first instructions (one dependent fetch less at the start of every launch).
FLAGS += ["-mllvm", "-amdgpu-kernarg-preload-count=16"]


def build(verbose: bool = True) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(HERE, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [hipcc, *FLAGS, "-c", os.path.join(HERE, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if out.strip() and verbose:
            print(out)
        if p.returncode != 0:
            failed = True
            print(f"hipcc failed on {src}", file=sys.stderr)
    if failed:
        raise RuntimeError("libflashstu_hip.so: compilation failed")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build())
