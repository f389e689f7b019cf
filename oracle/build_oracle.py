"""Compile the scalar C oracle (oracle/llmq_oracle.c) into oracle/liboracle.so with gcc.

Test infrastructure only.  The reference's own native path (CUDA + CUTLASS) cannot be
compiled in this image, so there is no oracle/_ref build.
"""
import pathlib
import subprocess

HERE = pathlib.Path(__file__).resolve().parent
SRC = HERE / "llmq_oracle.c"
OUT = HERE / "liboracle.so"


def build(force: bool = True) -> pathlib.Path:
    if OUT.exists() and not force and OUT.stat().st_mtime >= SRC.stat().st_mtime:
        return OUT
    cmd = ["gcc", "-O2", "-fPIC", "-shared", "-fno-fast-math", "-ffp-contract=off",
           "-o", str(OUT), str(SRC), "-lm"]
    subprocess.run(cmd, check=True)
    return OUT


if __name__ == "__main__":
    print(build())
