"""Compile the plain-C update oracle into ``oracle/libckv_oracle.so`` with gcc."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "ckv_oracle_update.c")
OUT = os.path.join(HERE, "libckv_oracle.so")


def build(force: bool = True) -> str:
    if not force and os.path.exists(OUT) and os.path.getmtime(OUT) >= os.path.getmtime(SRC):
        return OUT
    cmd = ["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-Wall", "-Wextra", "-o", OUT, SRC]
    subprocess.run(cmd, check=True, cwd=HERE)
    return OUT


if __name__ == "__main__":
    print(build())
