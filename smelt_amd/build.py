"""Builds the gfx950 code object and the C-ABI host library in-tree.

    python -m smelt_amd.build          # compile everything

Outputs (git-ignored, shipped to the GPU box as built files):
    smelt_amd/lib/smelt_kernels*.hsaco  hipcc --genco, gfx950 only, one per translation unit
    smelt_amd/lib/libsmelt_hip.so       host runtime + record emitters (links libamdhip64); carries one
                                        small gfx950 image of its own (static_scratch.hip)
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
HSACO = os.path.join(LIB, "smelt_kernels.hsaco")
# every translation unit under csrc/kernels becomes one code object; the runtime loads them all
KERNEL_UNITS = ["smelt_kernels", "smelt_kernels_batched_f16", "smelt_kernels_batched_bf16",
                "smelt_kernels_signed", "smelt_kernels_planes", "smelt_kernels_qmm",
                "smelt_kernels_layer", "smelt_kernels_mm1", "smelt_kernels_mm1f", "smelt_kernels_qms", "smelt_kernels_qmt"]
HOST_LIB = os.path.join(LIB, "libsmelt_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 instructions are switched off for all device code
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
HOST_SOURCES = ["runtime.cpp", "pipeline_table.cpp", "compiler.cpp", "import.cpp"]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("build step failed: " + " ".join(cmd))


def code_objects() -> list[str]:
    return [os.path.join(LIB, unit + ".hsaco") for unit in KERNEL_UNITS]


def build_kernels() -> list[str]:
    """Compiles the translation units side by side (one hipcc process each)."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(LIB, exist_ok=True)

    def one(unit: str) -> str:
        out = os.path.join(LIB, unit + ".hsaco")
        _run([HIPCC, *DEVICE_FLAGS, "--genco", "-o", out, os.path.join(CSRC, "kernels", unit + ".hip")])
        return out

    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        built = list(pool.map(one, KERNEL_UNITS))
    # the runtime loads exactly the code objects this build made
    with open(os.path.join(LIB, "smelt_kernels.manifest"), "w") as f:
        f.write("# code objects of this build, one per line\n")
        for unit in KERNEL_UNITS:
            f.write(unit + ".hsaco\n")
    return built


def build_host() -> str:
    os.makedirs(LIB, exist_ok=True)
    srcs = [os.path.join(CSRC, s) for s in HOST_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    # the one host-library source with device code in it: the file-scope scratch array, its fill
    # kernel and the entry point that uses them
    scratch_obj = os.path.join(LIB, "static_scratch.o")
    _run([HIPCC, *DEVICE_FLAGS, "-fPIC", "-c", "-o", scratch_obj, os.path.join(CSRC, "static_scratch.hip")])
    _run([os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
          "-D__HIP_PLATFORM_AMD__", f"-I{rocm}/include", "-o", HOST_LIB, *srcs, scratch_obj,
          f"-L{rocm}/lib", f"-Wl,-rpath,{rocm}/lib", "-lamdhip64", "-lpthread"])
    return HOST_LIB


def build_all() -> None:
    build_kernels()
    build_host()


if __name__ == "__main__":
    build_all()
    for path in code_objects():
        print(path)
    print(HOST_LIB)
