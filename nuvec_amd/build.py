"""Compiles the gfx950 kernels and the C ABI into `nuvec_amd/libnuvec_hip.so` with hipcc.

Cross-compiles without a GPU.  Run as `python -m nuvec_amd.build` or through
`__graft_entry__.build()`.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(HERE, "..", "include")
LIB = os.path.join(HERE, "libnuvec_hip.so")
SOURCES = ["qmf_b8.hip", "qmf_fp8.hip", "qmf_b6.hip", "qmf_b5.hip", "qmf_b4.hip", "qmf_fp4.hip", "qmf_nvfp4.hip", "qmf_b3.hip", "qmf_b2.hip", "qmf_b1.hip", "qmm.hip", "qmv.hip", "qmv_dot8.hip", "qmm_f32.hip", "qmr.hip",
           "qvm.hip", "nvq_api.hip", "affine_quant.hip", "fp_quant.hip", "qmf.hip", "gather.hip", "repack.hip", "calib.hip", "qattn.hip", "qmd.hip", "glu.hip"]  # slowest to compile first

# -ffp-contract=off: the quantizers must round every operation as the CPU does; fused
# multiply-adds are written explicitly where wanted.  Correctly rounded f32 division is
# hipcc's default and is spelled out because the bit-exact quantizers depend on it.
# Packed-FP32 instructions are switched off for all device code.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-gpu-flush-denormals-to-zero",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-inline-asm", "-fvisibility=hidden",
    f"-I{INCLUDE}", f"-I{CSRC}",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def build(verbose: bool = False, jobs: int = 8, changed_only: bool = False) -> str:
    """Compiles every source and links the library.  `changed_only` (a development aid, `--changed` on the command line):
    sources older than their object files are not compiled again, unless a header is newer than the object."""
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    headers = [os.path.join(d, f) for d in (CSRC, INCLUDE) for f in os.listdir(d) if f.endswith(".h")]
    newest_header = max(os.path.getmtime(h) for h in headers)

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        if changed_only and os.path.exists(obj) and os.path.getmtime(obj) > max(newest_header, os.path.getmtime(os.path.join(CSRC, src))):
            return obj
        cmd = [hipcc, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}\n{proc.stderr}")
        # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless.
        noise = "is not a recognized feature for this target"
        err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l and l.strip())
        if verbose and err:
            print(err, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, changed_only="--changed" in sys.argv))
