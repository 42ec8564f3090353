"""Build tests/c_abi/spmv_from_c.cpp (a C++ caller of the two C interfaces) into tests/c_abi/_build/."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

SOURCE = os.path.join(HERE, "spmv_from_c.cpp")
BINARY = os.path.join(HERE, "_build", "spmv_from_c")


def build(force: bool = False) -> str:
    from flexspmv_amd.build import INCLUDE_DIR, hipcc_path
    if not force and os.path.exists(BINARY) and os.path.getmtime(BINARY) >= os.path.getmtime(SOURCE):
        return BINARY
    os.makedirs(os.path.dirname(BINARY), exist_ok=True)
    cmd = [hipcc_path(), "-O2", "-std=c++17", f"-I{INCLUDE_DIR}", SOURCE, "-o", BINARY, "-ldl"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"building {SOURCE} failed:\n{' '.join(cmd)}\n{proc.stdout}")
    return BINARY


if __name__ == "__main__":
    print(build(force=True))
