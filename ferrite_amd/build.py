"""Builds libferrite_amd.so in-tree: the gfx950 code objects (hipcc --genco), linked into the host library as data.

    python -m ferrite_amd.build        # compile everything
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
KERN = os.path.join(CSRC, "kernels")
OUT = os.path.join(HERE, "_build")
LIB = os.path.join(HERE, "libferrite_amd.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")

# -packed-fp32-ops off: the compiler must not form v_pk_*_f32 from the float code in these kernels
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-mcode-object-version=5",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
KERNELS = ["k_exl3", "k_fp4", "k_route", "k_bf16"]
HOST = ["fe_hip.cpp", "fe_exl3.cpp", "fe_fp4.cpp", "fe_bf16.cpp", "fe_route.cpp"]
# host sources that also hold device code (a file-scope __device__ array): compiled by hipcc as one unit
HOST_HIP = ["fe_exl3_static.hip"]


def _run(cmd, **kw):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, **kw)
    if r.returncode:
        sys.stderr.write(" ".join(cmd) + "\n" + r.stdout)
        raise RuntimeError(f"build step failed: {cmd[0]} ... {cmd[-1]}")
    return r.stdout


def build(verbose: bool = False) -> str:
    os.makedirs(OUT, exist_ok=True)
    only = [k for k in os.environ.get("FE_BUILD_ONLY", "").split(",") if k]  # e.g. k_exl3: the others are kept as built
    inc = ["-I", os.path.join(os.path.dirname(HERE), "include"), "-I", CSRC, "-I", os.path.join(ROCM, "include")]
    jobs = []
    for k in KERNELS:
        if only and k not in only and os.path.exists(os.path.join(OUT, k + ".hsaco")):
            continue
        jobs.append([HIPCC, "--genco", "--no-gpu-bundle-output", *DEVICE_FLAGS, "-I", KERN, os.path.join(KERN, k + ".hip"),
                     "-o", os.path.join(OUT, k + ".hsaco")])
    for src in HOST_HIP:
        jobs.append([HIPCC, "-c", "-fPIC", *DEVICE_FLAGS, *inc, os.path.join(CSRC, src), "-o",
                     os.path.join(OUT, src.replace(".hip", ".o"))])
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        list(pool.map(_run, jobs))
    # the code objects become .rodata of the library (.incbin resolves against the working directory)
    _run(["gcc", "-c", os.path.join(CSRC, "fe_embed.S"), "-o", os.path.join(OUT, "fe_embed.o")], cwd=OUT)
    objs = [os.path.join(OUT, "fe_embed.o")] + [os.path.join(OUT, s.replace(".hip", ".o")) for s in HOST_HIP]
    for src in HOST:
        o = os.path.join(OUT, src.replace(".cpp", ".o"))
        _run(["g++", "-c", "-O2", "-fPIC", "-std=c++17", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__", *inc,
              os.path.join(CSRC, src), "-o", o])
        objs.append(o)
    _run(["g++", "-shared", "-o", LIB, *objs, "-L", os.path.join(ROCM, "lib"), "-lamdhip64",
          "-Wl,-rpath," + os.path.join(ROCM, "lib"), "-Wl,--no-undefined"])
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(verbose=True)
