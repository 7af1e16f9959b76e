"""Builds ``libf8oracle.so`` from ``f8_oracle.c`` with gcc (test infrastructure)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "f8_oracle.c")
LIB = os.path.join(HERE, "libf8oracle.so")


def build(force: bool = True) -> str:
    if not force and os.path.exists(LIB) and os.path.getmtime(LIB) >= os.path.getmtime(SRC):
        return LIB
    cmd = ["gcc", "-O2", "-fno-fast-math", "-ffp-contract=off", "-shared", "-fPIC", "-o", LIB, SRC, "-lm"]
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build())
