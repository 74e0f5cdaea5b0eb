"""Builds libllmopt_hip.so (gfx950) in-tree with hipcc.

    python -m llmopt_amd.build [--force] [--host-ubsan]

The shared library holds the HIP kernels and the flat C ABI declared in
include/llmopt_hip.h.  hipcc cross-compiles without a GPU.

--host-ubsan builds a second library, libllmopt_hip_ubsan.so, whose HOST code (the runtime, the
retained plans, the entry points, the operator mirror, the sampler) traps on undefined behaviour
and out-of-bounds array indices; the GPU code is the same.  Run the tests against it with
LLMOPT_HIP_LIBRARY=llmopt_amd/libllmopt_hip_ubsan.so: a trap ends the process with SIGILL.
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
UBSAN_BUILD = os.path.join(CSRC, "build", "ubsan")
UBSAN_LIBRARY = os.path.join(HERE, "libllmopt_hip_ubsan.so")
# host pass only (each -fsanitize option directly behind -Xarch_host): no runtime library needed
HOST_UBSAN = ["-Xarch_host", "-fsanitize=undefined,bounds", "-Xarch_host", "-fsanitize-trap=undefined,bounds"]

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


def _compile(source: str, force: bool, host_ubsan: bool = False) -> str:
    rel = os.path.relpath(source, CSRC).replace(os.sep, "_")
    host_ubsan = host_ubsan and source.endswith(".cpp")  # kernel files: the ordinary objects
    obj = os.path.join(UBSAN_BUILD if host_ubsan else BUILD, rel + ".o")
    newest_dep = max(os.path.getmtime(p) for p in [source, os.path.abspath(__file__)] + _headers())
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= newest_dep:
        return obj
    command = ["hipcc", *COMMON, *PER_FILE.get(os.path.basename(source), []), *(HOST_UBSAN if host_ubsan else []),
               "-c", source, "-o", obj]
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


def build(force: bool = False, host_ubsan: bool = False) -> str:
    os.makedirs(UBSAN_BUILD if host_ubsan else BUILD, exist_ok=True)
    library = UBSAN_LIBRARY if host_ubsan else LIBRARY
    with concurrent.futures.ThreadPoolExecutor(max_workers=6) as pool:
        objects = list(pool.map(lambda s: _compile(s, force, host_ubsan), sources()))
    newest = max(os.path.getmtime(o) for o in objects)
    if force or not os.path.exists(library) or os.path.getmtime(library) < newest:
        command = ["hipcc", "-shared", "-fPIC", "--offload-arch=gfx950", "-fno-gpu-sanitize",
                   "-o", library, *objects]
        result = subprocess.run(command, capture_output=True, text=True)
        if result.returncode != 0:
            raise RuntimeError(f"link failed:\n{result.stderr}")
    return library


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, host_ubsan="--host-ubsan" in sys.argv))
