"""Build the two native libraries of the package in-tree.

* ``cera_amd/lib/libcera_hip.so``  -- HIP kernels + C-ABI (hipcc, gfx950)
* ``cera_amd/lib/libcera_host.so`` -- CPU host layer: quantizers, GGUF, synthetic models (g++)
* ``cera_amd/lib/libcera_hip_llama.so`` + ``cera_amd/lib/cera-hip`` -- the Model-trait layer
  above the C-ABI and its command-line driver (g++)
"""
from __future__ import annotations

import os
import shutil
import subprocess
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
LIB_DIR = PKG / "lib"
HIP_LIB = LIB_DIR / "libcera_hip.so"
HOST_LIB = LIB_DIR / "libcera_host.so"
LLAMA_LIB = LIB_DIR / "libcera_hip_llama.so"
CLI_BIN = LIB_DIR / "cera-hip"
HSACO = LIB_DIR / "cera_hip_gfx950.hsaco"

HIP_SRCS = sorted((PKG / "csrc").glob("*.hip"))
HOST_SRCS = sorted((PKG / "host").glob("*.cpp"))

# -ffp-contract=off: the parity target never fuses a*b+c implicitly; FMAs in
# the kernels are spelled fmaf().  The packed-fp32 feature is switched off
# because some packed forms have produced wrong results on this hardware pool.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results straight into VGPRs: the GEMM epilogue consumes every accumulator element
    # on the VALU, and the AGPR form would cost one v_accvgpr_read per element on top
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wall", "-Wno-unused-function",
]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off", "-fno-fast-math",
              "-pthread", "-Wall", "-Wextra", "-fvisibility=hidden"]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found")


def build_hip(verbose: bool = False, jobs: int = 8) -> Path:
    """Compile every csrc/*.hip to an object (in parallel) and link the C-ABI library."""
    from concurrent.futures import ThreadPoolExecutor

    LIB_DIR.mkdir(exist_ok=True)
    obj_dir = LIB_DIR / "obj"
    obj_dir.mkdir(exist_ok=True)
    srcs = sorted((PKG / "csrc").glob("*.hip"))
    hipcc = hipcc_path()
    flags = [f for f in HIPCC_FLAGS if f != "-shared"]

    def compile_one(src: Path):
        obj = obj_dir / (src.stem + ".o")
        cmd = [hipcc, *flags, f"-I{ROOT / 'include'}", f"-I{PKG / 'csrc'}", "-c", str(src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        return src, obj, cmd, r

    objs = []
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        for src, obj, cmd, r in ex.map(compile_one, srcs):
            if verbose or r.returncode:
                print(" ".join(cmd))
                print(r.stdout + r.stderr)
            if r.returncode:
                raise RuntimeError(f"hipcc failed on {src.name}")
            objs.append(str(obj))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", str(HIP_LIB)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or r.returncode:
        print(" ".join(cmd))
        print(r.stdout + r.stderr)
    if r.returncode:
        raise RuntimeError("hipcc link failed")
    return HIP_LIB


def build_hsaco(verbose: bool = False) -> Path:
    """The standalone gfx950 code object of the lower ABI (include/cera_hip_kernels.h)."""
    LIB_DIR.mkdir(exist_ok=True)
    flags = [f for f in HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    cmd = [hipcc_path(), "--genco", "--no-gpu-bundle-output", *flags, f"-I{ROOT / 'include'}", f"-I{PKG / 'csrc'}",
           str(PKG / "csrc" / "lower" / "cera_hip_gfx950.hip"), "-o", str(HSACO)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or r.returncode:
        print(" ".join(cmd))
        print(r.stdout + r.stderr)
    if r.returncode:
        raise RuntimeError("hipcc --genco failed")
    return HSACO


def build_host(verbose: bool = False) -> Path:
    LIB_DIR.mkdir(exist_ok=True)
    srcs = sorted((PKG / "host").glob("*.cpp"))
    cmd = ["g++", *HOST_FLAGS, f"-I{ROOT / 'include'}", f"-I{PKG / 'host'}", *map(str, srcs),
           "-o", str(HOST_LIB), "-ldl"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or r.returncode:
        print(" ".join(cmd))
        print(r.stdout + r.stderr)
    if r.returncode:
        raise RuntimeError("g++ failed building the host library")
    return HOST_LIB


def build_backend(verbose: bool = False) -> Path:
    """HipLlamaModel + its C face (libcera_hip_llama.so) and the cera-hip driver binary.

    Both link against the two libraries above, found at run time next to themselves.
    """
    common = ["g++", "-O2", "-std=c++17", "-fPIC", "-pthread", "-Wall", "-Wextra", "-fvisibility=hidden",
              f"-I{ROOT / 'include'}", f"-I{PKG / 'host'}", f"-I{PKG / 'backend'}"]
    link = [f"-L{LIB_DIR}", "-lcera_hip", "-lcera_host", "-Wl,-rpath,$ORIGIN"]
    b = PKG / "backend"
    gguf = str(PKG / "host" / "gguf.cpp")  # C++ classes are not exported by the host library: compile them in
    cmds = [
        [*common, "-shared", str(b / "hip_llama.cpp"), str(b / "hip_llama_capi.cpp"), gguf, "-o", str(LLAMA_LIB),
         *link],
        [*common, str(b / "cli.cpp"), str(b / "hip_llama.cpp"), gguf, "-o", str(CLI_BIN), *link],
    ]
    for cmd in cmds:
        r = subprocess.run(cmd, capture_output=True, text=True)
        if verbose or r.returncode:
            print(" ".join(cmd))
            print(r.stdout + r.stderr)
        if r.returncode:
            raise RuntimeError("g++ failed building the backend layer")
    return LLAMA_LIB


def build_all(verbose: bool = False) -> None:
    build_host(verbose)
    build_hip(verbose)
    build_hsaco(verbose)
    build_backend(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
