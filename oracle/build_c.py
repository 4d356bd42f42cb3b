"""Recipe for the C restatement (test infrastructure): gcc, in-tree output oracle/liboracle_c.so."""

from __future__ import annotations

import shutil
import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
SRC = HERE / "oracle_c.c"
LIB = HERE / "liboracle_c.so"


def build_oracle_c() -> Path:
    gcc = shutil.which("gcc")
    if gcc is None:
        raise RuntimeError("gcc not found: the C restatement of the oracle cannot be built")
    cmd = [gcc, "-O2", "-std=c11", "-fPIC", "-shared", "-fno-fast-math", "-o", str(LIB), str(SRC), "-lm"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"gcc failed on {SRC.name}:\n{res.stdout}\n{res.stderr}")
    return LIB


if __name__ == "__main__":
    print(build_oracle_c())
