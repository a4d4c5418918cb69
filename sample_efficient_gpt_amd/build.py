"""Builds libsegpt_attn.so (gfx950) in-tree with hipcc.  `python -m sample_efficient_gpt_amd.build`."""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(os.path.dirname(PKG_DIR), "include")
LIB_PATH = os.path.join(PKG_DIR, "libsegpt_attn.so")
SOURCES = ["api.hip", "f32_path.hip", "pre_post.hip", "fwd_mfma.hip", "bwd_mfma.hip", "decode_mfma.hip"]
# Per-source flags.  The forward never needs more than 256 registers, but at head_dim 128 it runs one
# workgroup per CU and the compiler would then move every MFMA result into the accumulation registers
# (one v_accvgpr_read per score before exp2); keeping the ordinary-register form is 8 % faster there.
# The forward is also scheduled with the backend's "max-ilp" strategy (2-4 % faster in same-box A/B runs; no effect
# on the backward kernels, which keep the default).
EXTRA_FLAGS = {"fwd_mfma.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1", "-mllvm", "-amdgpu-sched-strategy=max-ilp"],
               "decode_mfma.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}

# -packed-fp32-ops is switched off: hipcc -O3 otherwise forms v_pk_*_f32 from ordinary float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-ignored-attributes", "-Wno-unknown-warning-option",
    "-Wno-int-to-pointer-cast",  # host pass only: LDS addresses are 32-bit integers on the device
    f"-I{INCLUDE}", f"-I{CSRC}",
]


def _hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (needs ROCm; looked on PATH and in /opt/rocm/bin)")


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    return out


def build(verbose: bool = False, extra_flags: list[str] | None = None) -> str:
    """Compile every HIP source and link the shared library; returns its path."""
    hipcc = _hipcc()
    obj_dir = os.path.join(PKG_DIR, "build")
    os.makedirs(obj_dir, exist_ok=True)
    flags = HIPCC_FLAGS + (extra_flags or [])

    def compile_one(src):
        obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
        out = _run([hipcc, *flags, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out:
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    tmp = LIB_PATH + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", tmp])
    os.replace(tmp, LIB_PATH)
    if verbose:
        print("built", LIB_PATH)
    # stand-alone measurement programs (not part of the library): one executable per source under csrc/microbench
    mb_dir = os.path.join(CSRC, "microbench")
    for src in sorted(f for f in os.listdir(mb_dir) if f.endswith(".hip")):
        exe = os.path.join(PKG_DIR, src.replace(".hip", ".bin"))
        _run([hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
              "-Wno-unused-command-line-argument", os.path.join(mb_dir, src), "-o", exe + ".tmp"])
        os.replace(exe + ".tmp", exe)
        if verbose:
            print("built", exe)
    return LIB_PATH


if __name__ == "__main__":
    build(verbose=True, extra_flags=sys.argv[1:])
