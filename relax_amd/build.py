"""Builds ``librelax_amd.so`` (hand-written gfx950 HIP kernels + C ABI) in-tree with hipcc.

Run as ``python relax_amd/build.py``.  The library is written next to this file so it travels with the source tree.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
BUILD_DIR = os.path.join(HERE, "csrc", "build")
LIB_PATH = os.path.join(HERE, "librelax_amd.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # packed-fp32 VALU forms are kept off on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _file_flags(src: str) -> list[str]:
    """Extra compiler flags a source file asks for itself, on ``// hipcc-flags: ...`` lines of its leading comment."""
    flags: list[str] = []
    with open(src) as f:
        for line in f:
            if not line.startswith("//"):
                break
            if line.startswith("// hipcc-flags:"):
                flags += line[len("// hipcc-flags:"):].split()
    return flags


def _compile(src: str) -> str:
    obj = os.path.join(BUILD_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, *_file_flags(src), "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    noise = "is not a recognized feature for this target"
    warn = "\n".join(l for l in r.stderr.splitlines() if noise not in l and l.strip())
    if "warning" in warn:
        sys.stderr.write(warn + "\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(BUILD_DIR, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources")
    build_abi_client(verbose)
    return LIB_PATH


ABI_CLIENT_SRC = os.path.join(os.path.dirname(HERE), "tests", "abi_client.c")
ABI_CLIENT = os.path.join(BUILD_DIR, "abi_client")


def build_abi_client(verbose: bool = True) -> str | None:
    """The plain-C client of the library used by the GPU tests (no Python, no PyTorch in the process): compiled as C
    against ``include/relax_amd.h`` and the HIP runtime API, linked to the library just built."""
    if not os.path.exists(ABI_CLIENT_SRC):
        return None
    rocm = os.path.dirname(os.path.dirname(HIPCC))
    cmd = ["gcc", "-std=c11", "-O1", "-Wall", "-D__HIP_PLATFORM_AMD__", f"-I{INCLUDE}", f"-I{rocm}/include",
           ABI_CLIENT_SRC, "-o", ABI_CLIENT, f"-L{HERE}", "-lrelax_amd", f"-L{rocm}/lib", "-lamdhip64", "-lm",
           f"-Wl,-rpath,{HERE}", "-Wl,-rpath,$ORIGIN/../..", f"-Wl,-rpath,{rocm}/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"building the C client failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {ABI_CLIENT}")
    return ABI_CLIENT


if __name__ == "__main__":
    build()
