"""Compiles the C restatement of the oracle (mxfp4_ref.c) with gcc.  Test infrastructure only."""

from __future__ import annotations

import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
OUT = HERE / "_build" / "libmxfp4_ref.so"


def build_oracle() -> Path:
    OUT.parent.mkdir(exist_ok=True)
    subprocess.run(["gcc", "-O2", "-shared", "-fPIC", "-o", str(OUT), str(HERE / "mxfp4_ref.c"), "-lm"], check=True)
    return OUT


if __name__ == "__main__":
    print(build_oracle())
