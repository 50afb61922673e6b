"""Build recipe for libsngguf.so (hipcc, gfx950 only).

``python -m sensenova_u1_amd.build`` (or ``build_library()``) compiles every source under
``csrc/`` and links the in-tree ``libsngguf.so`` next to this file.  hipcc cross-compiles
without a GPU, so this runs on a CPU-only build host; the GPU side only loads the result.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libsngguf.so")
SOURCES = ["api.cpp", "gguf_reader.cpp", "dequantize.hip", "plain_bf16.hip", "rmsnorm.hip", "gemv.hip", "gemv_q8_mfma.hip", "gemv_kq_mfma.hip", "gemv_q8_tiled.hip", "gemm.hip", "gemm_tiles.hip", "gemm_dense4.hip", "static_scratch.hip", "stream_probe.hip"]

# packed-fp32 VALU forms are switched off for every device compile of this library
HIP_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-Wall",
    # no fused multiply-add unless written as one: the fp16 decode chain rounds after every op
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the copy requests written as instructions name M0 as clobbered, which the compiler reports once per request
    "-Wno-inline-asm",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: libsngguf.so can only be built with the ROCm toolchain")
    return exe


# per-source additions.  gemv_kq_mfma.hip widens fp16 to fp32 with matrix instructions whose
# results the vector ALU consumes at once: they must land in ordinary VGPRs, not in accumulation
# registers that need one v_accvgpr_read per value.
SOURCE_FLAGS = {"gemv_kq_mfma.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def _compile(src: str, obj: str, extra: list[str]) -> None:
    cmd = [_hipcc(), *HIP_FLAGS, *SOURCE_FLAGS.get(src, []), *extra, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    noise = "unknown target feature"  # hipcc's host pass does not know the device-only feature flag
    warn = "\n".join(l for l in res.stderr.splitlines() if l.strip() and noise not in l and "packed-fp32-ops" not in l)
    if "warning" in warn:
        sys.stderr.write(warn + "\n")


def build_library(force: bool = True, extra_flags: list[str] | None = None, jobs: int = 4) -> str:
    """Compile and link libsngguf.so; returns its path.  ``force=False`` skips an up-to-date library."""
    srcs = [os.path.join(CSRC, s) for s in SOURCES] + [os.path.join(CSRC, "sngguf_common.hpp"), os.path.join(CSRC, "gemm_args.hpp"),
                                                        os.path.join(PKG_DIR, "..", "include", "sngguf.h")]
    if not force and os.path.exists(LIB_PATH) and all(os.path.getmtime(LIB_PATH) >= os.path.getmtime(s) for s in srcs):
        return LIB_PATH
    objdir = os.path.join(PKG_DIR, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, os.path.splitext(s)[0] + ".o") for s in SOURCES]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda so: _compile(so[0], so[1], extra_flags or []), zip(SOURCES, objs)))
    tmp = LIB_PATH + ".tmp"
    res = subprocess.run([_hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-pthread", "-o", tmp, *objs],
                         capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(force=True))
