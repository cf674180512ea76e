"""Compile oracle/rope_ring_ref.c (test infrastructure: the C restatement
that pins the PyTorch oracle) into oracle/_build/libsdv2_ref.so with gcc."""
import os
import shutil
import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
LIB = HERE / "_build" / "libsdv2_ref.so"


def build() -> Path:
    gcc = shutil.which("gcc")
    if gcc is None:
        raise RuntimeError("gcc not found")
    LIB.parent.mkdir(exist_ok=True)
    tmp = LIB.with_suffix(".so.tmp")
    subprocess.run([gcc, "-O2", "-std=c99", "-Wall", "-Wextra", "-Werror", "-ffp-contract=off", "-fPIC", "-shared",
                    str(HERE / "rope_ring_ref.c"), "-o", str(tmp)], check=True)
    os.replace(tmp, LIB)
    return LIB


if __name__ == "__main__":
    print(build())
