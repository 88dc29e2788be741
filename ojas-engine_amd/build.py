"""Offline build of the backend: gfx950 code objects (one per kernel family) and libojas_hip.so.

    python ojas-engine_amd/build.py            # build everything that is out of date
    python ojas-engine_amd/build.py --force    # rebuild everything

hipcc cross-compiles for gfx950 without a GPU.  Outputs stay in-tree (`hsaco/`, `libojas_hip.so`)
so they travel with the source tree to the machine that has the GPU.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
KERNELS = os.path.join(CSRC, "kernels")
HSACO = os.path.join(HERE, "hsaco")
LIB = os.path.join(HERE, "libojas_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

# Packed-FP32 instructions stay off for all device code on this target.
DEVICE_FLAGS = ["-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-Wno-unused-command-line-argument"]

# family -> (source, extra flags).  The decoder family and the GEMM's in-tile decoder must round
# every operation separately (no fused multiply-add).  OJK_ASM_FIRST_DOT: the three-operand first dot of a chain
# (ojk_common.h), where it was measured to pay.
FAMILIES = {
    "dequant": ("dequant.hip", ["-ffp-contract=off"]),
    "gemv": ("gemv.hip", []),
    "gemv_q8k": ("gemv_q8k.hip", ["-DOJK_ASM_FIRST_DOT"]),
    "glue": ("glue.hip", []),
    "gemm": ("gemm.hip", ["-ffp-contract=off"]),
    "gemm_xl": ("gemm_xl.hip", ["-ffp-contract=off"]),
    "gemm_q8k": ("gemm_q8k.hip", []),
    "moe": ("moe.hip", ["-DOJK_ASM_FIRST_DOT"]),
    "moe_iq": ("moe_iq.hip", []),
    "rowq8": ("rowq8.hip", ["-ffp-contract=off"]),
    "q80_dp4a": ("q80_dp4a.hip", []),
    "iq_grid": ("iq_grid.hip", ["-ffp-contract=off"]),
    "chain": ("chain.hip", []),
    "gemv_q8": ("gemv_q8.hip", ["-ffp-contract=off"]),
}

HOST_SOURCES = ["ojh_runtime.cpp", "ojh_manifest.cpp", "ojh_ops.cpp", "ojh_moe.cpp", "ojh_gguf.cpp", "ojh_expert_cache.cpp", "ojh_noalloc.cpp", "ojh_chain.cpp"]


def _newer(target: str, deps: list[str]) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps if os.path.exists(d))


def _run(cmd: list[str]) -> None:
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + r.stdout)
        raise RuntimeError(f"build step failed: {cmd[0]} ... {cmd[-1]}")


def build_kernels(force: bool = False) -> list[str]:
    os.makedirs(HSACO, exist_ok=True)
    headers = [os.path.join(KERNELS, f) for f in os.listdir(KERNELS) if f.endswith(".h")]
    out = []
    for family, (src, extra) in FAMILIES.items():
        srcp = os.path.join(KERNELS, src)
        if not os.path.exists(srcp):
            continue
        dst = os.path.join(HSACO, family + ".hsaco")
        if force or _newer(dst, [srcp] + headers):
            _run([HIPCC, f"--offload-arch={ARCH}", "--genco", *DEVICE_FLAGS, *extra, "-o", dst, srcp])
        out.append(dst)
    return out


def build_library(force: bool = False) -> str:
    srcs = [os.path.join(CSRC, s) for s in HOST_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    deps = srcs + [os.path.join(CSRC, "ojh_internal.h"), os.path.join(HERE, "..", "include", "ojas_hip.h"),
                   os.path.join(KERNELS, "ojk_chain.h")]
    if force or _newer(LIB, deps):
        _run([HIPCC, f"--offload-arch={ARCH}", *DEVICE_FLAGS, "-fPIC", "-shared", "-Wall", "-o", LIB, *srcs, "-ldl"])
    return LIB


def build_all(force: bool = False) -> None:
    build_kernels(force)
    build_library(force)


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
    print("built:", LIB, "and", ", ".join(sorted(os.listdir(HSACO))))
