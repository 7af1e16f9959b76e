"""Compiles csrc/*.hip into libf8mi.so for gfx950 with hipcc (no GPU needed)."""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libf8mi.so")
# bench-only helper (register-only MFMA loop), kept out of libf8mi.so: it synchronises and copies from the host
PROBE_SRC = os.path.join(CSRC, "bench", "f8mi_probe.hip")
PROBE_LIB = os.path.join(HERE, "libf8mi_probe.so")
OBJ_DIR = os.path.join(CSRC, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    subprocess.run([HIPCC, *FLAGS, "-c", src, "-o", obj], check=True)
    return obj


def build(verbose: bool = True) -> str:
    """Always recompiles every source and relinks the shared library."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs], check=True)
    subprocess.run([HIPCC, *FLAGS, "-shared", PROBE_SRC, "-o", PROBE_LIB], check=True)
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources", file=sys.stderr)
    return LIB


if __name__ == "__main__":
    build()
