"""Recipe for the plain-C caller of the library (test infrastructure): gcc, in-tree output
tests/c_abi/abi_caller, linked against the in-tree library and the HIP runtime."""

from __future__ import annotations

import shutil
import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
ROOT = HERE.parents[1]
SRC = HERE / "abi_caller.c"
EXE = HERE / "abi_caller"
ROCM = Path("/opt/rocm")


def build_abi_caller() -> Path:
    gcc = shutil.which("gcc")
    if gcc is None:
        raise RuntimeError("gcc not found: the C caller cannot be built")
    libdir = ROOT / "triturus_amd" / "lib"
    cmd = [
        gcc, "-std=c11", "-O2", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__",
        f"-I{ROCM / 'include'}", f"-I{ROOT / 'include'}", str(SRC), "-o", str(EXE),
        f"-L{libdir}", "-ltriturus_hip", f"-L{ROCM / 'lib'}", "-lamdhip64",
        "-Wl,-rpath,$ORIGIN/../../triturus_amd/lib", f"-Wl,-rpath,{ROCM / 'lib'}",
    ]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"gcc failed on {SRC.name}:\n{res.stdout}\n{res.stderr}")
    return EXE


if __name__ == "__main__":
    print(build_abi_caller())
