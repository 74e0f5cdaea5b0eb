"""Builds libllmopt_hip.so (gfx950) in-tree with hipcc.

    python -m llmopt_amd.build [--force]

The shared library holds the HIP kernels and the flat C ABI declared in
include/llmopt_hip.h.  hipcc cross-compiles without a GPU.
"""
from __future__ import annotations

import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
BUILD = os.path.join(CSRC, "build")
LIBRARY = os.path.join(HERE, "libllmopt_hip.so")

# -packed-fp32-ops off: hipcc must not form v_pk_*_f32 on this pool.
COMMON = ["-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-Wall", "-Wno-unused-function", "-fno-gpu-sanitize"]


# Kernels whose MFMA accumulators are also rescaled by vector instructions (online softmax):
# with the accumulators in AGPRs the compiler copies every one of them to a VGPR and back on
# each loop iteration, so these files keep them in VGPRs.  (The GEMM kernels want the AGPRs:
# their accumulators are touched by MFMAs only and the VGPRs are needed for everything else.)
PER_FILE = {
    "dense_attention.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "q8_attention.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}


def sources() -> list[str]:
    found = sorted(glob.glob(os.path.join(CSRC, "*.cpp")))
    found += sorted(glob.glob(os.path.join(CSRC, "host", "*.cpp")))
    found += sorted(glob.glob(os.path.join(CSRC, "kernels", "*.hip")))
    return found


def _headers() -> list[str]:
    found = glob.glob(os.path.join(CSRC, "**", "*.h"), recursive=True)
    found += glob.glob(os.path.join(HERE, "..", "include", "*.h"))
    return found


def _compile(source: str, force: bool) -> str:
    rel = os.path.relpath(source, CSRC).replace(os.sep, "_")
    obj = os.path.join(BUILD, rel + ".o")
    newest_dep = max(os.path.getmtime(p) for p in [source, os.path.abspath(__file__)] + _headers())
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= newest_dep:
        return obj
    command = ["hipcc", *COMMON, *PER_FILE.get(os.path.basename(source), []), "-c", source, "-o", obj]
    if source.endswith(".cpp"):
        command[1:1] = ["-x", "hip"]
    result = subprocess.run(command, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    stderr = "\n".join(line for line in result.stderr.splitlines() if noise not in line)
    if result.returncode != 0:
        raise RuntimeError(f"hipcc failed for {source}:\n{stderr}")
    if stderr.strip():
        sys.stderr.write(stderr + "\n")
    return obj


def build(force: bool = False) -> str:
    os.makedirs(BUILD, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=6) as pool:
        objects = list(pool.map(lambda s: _compile(s, force), sources()))
    newest = max(os.path.getmtime(o) for o in objects)
    if force or not os.path.exists(LIBRARY) or os.path.getmtime(LIBRARY) < newest:
        command = ["hipcc", "-shared", "-fPIC", "--offload-arch=gfx950", "-fno-gpu-sanitize",
                   "-o", LIBRARY, *objects]
        result = subprocess.run(command, capture_output=True, text=True)
        if result.returncode != 0:
            raise RuntimeError(f"link failed:\n{result.stderr}")
    return LIBRARY


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
