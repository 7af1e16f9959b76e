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


def _compile(src: str, obj_dir: str = OBJ_DIR, defines=()) -> str:
    obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
    subprocess.run([HIPCC, *FLAGS, *defines, "-c", src, "-o", obj], check=True)
    return obj


def build(verbose: bool = True, out: str = LIB, defines=()) -> str:
    """Always recompiles every source and relinks the shared library.  ``out`` / ``defines`` (-DNAME=value flags) make a
    measurement build beside the shipped one (load it by pointing F8MI_LIB at it); its objects go to their own folder."""
    obj_dir = OBJ_DIR if out == LIB else os.path.join(OBJ_DIR, os.path.basename(out) + ".objs")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(lambda src: _compile(src, obj_dir, tuple(defines)), srcs))
    subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out, *objs], check=True)
    if out == LIB:
        subprocess.run([HIPCC, *FLAGS, "-shared", PROBE_SRC, "-o", PROBE_LIB], check=True)
    if verbose:
        print(f"built {out} from {len(srcs)} sources", file=sys.stderr)
    return out


if __name__ == "__main__":
    import argparse

    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--out", default=LIB, help="path of the shared library to write (default: the in-tree libf8mi.so)")
    ap.add_argument("-D", dest="defines", action="append", default=[], metavar="NAME=value",
                    help="preprocessor definition for a measurement build, e.g. -DF8MI_WALK_GROUP=2")
    a = ap.parse_args()
    build(out=os.path.abspath(a.out), defines=["-D" + d for d in a.defines])
