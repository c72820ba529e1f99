"""Compiles the HIP library (and the C++ adapter's test driver) for gfx950, in-tree."""
from __future__ import annotations

import shutil
import subprocess
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent
ROOT = PACKAGE_DIR.parent
CSRC = PACKAGE_DIR / "csrc"
HOST = PACKAGE_DIR / "host"
LIB_DIR = PACKAGE_DIR / "lib"

HIP_SOURCES = ["capi.hip", "kquant_gemv.hip", "f32_gemv.hip", "kquant_gemm_mfma.hip",
               "moe.hip", "aux_kernels.hip"]
# -packed-fp32-ops off: no v_pk_*_f32 is generated.  -ffp-contract=off: fused
# multiply-adds happen only where the source writes them, so the arithmetic of a
# token column is the same in every kernel instantiation.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wextra"]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in proc.stdout.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if out.strip():
        print(out)


def build_library() -> Path:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    LIB_DIR.mkdir(exist_ok=True)
    target = LIB_DIR / "libgufo_hip.so"
    _run([hipcc, *HIP_FLAGS, "-shared", "-o", str(target),
          *[str(CSRC / s) for s in HIP_SOURCES]])
    return target


def build_host_tests() -> list[Path]:
    """The C++ adapter's own test program (plain main(), like the reference's tests).
    It links the library and, as its checker, the CPU restatement in oracle/."""
    source = HOST / "hip_projections_test.cpp"
    oracle_dir = ROOT / "oracle"
    subprocess.run(["make", "-s", "-C", str(oracle_dir), "all"], check=True)
    target = LIB_DIR / "hip_projections_test"
    _run(["g++", "-std=c++20", "-O2", "-mf16c", "-Wall", "-Wextra", "-I", str(ROOT / "include"),
          "-I", str(HOST), "-I", str(oracle_dir), "-o", str(target), str(source),
          str(HOST / "hip_projections.cpp"), "-L", str(LIB_DIR), "-lgufo_hip",
          "-L", str(oracle_dir), "-lkquant_oracle",
          "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,$ORIGIN/../../oracle", "-pthread"])
    return [target]


def build_model_library() -> Path:
    """The host side above the C-ABI as a library of its own: the GGUF reader, the stage
    table, the Projections adapter and their extern "C" layer (include/gufo_hip_model.h).
    Host code only (g++); links libgufo_hip.so."""
    target = LIB_DIR / "libgufo_hip_model.so"
    _run(["g++", "-std=c++20", "-O2", "-mf16c", "-fPIC", "-shared", "-Wall", "-Wextra",
          "-I", str(ROOT / "include"), "-I", str(HOST), "-o", str(target),
          str(HOST / "model_capi.cpp"), str(HOST / "gguf_model.cpp"),
          str(HOST / "hip_projections.cpp"), "-L", str(LIB_DIR), "-lgufo_hip",
          "-Wl,-rpath,$ORIGIN", "-pthread"])
    return target


def build_all() -> None:
    build_library()
    build_model_library()
    build_host_tests()


if __name__ == "__main__":
    build_all()
