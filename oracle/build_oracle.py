"""TEST INFRASTRUCTURE ONLY -- build recipes for the CPU oracle.

* ``build_graph_oracle(ir)``  g++ -O3 -fopenmp the generated oracle of a sub-graph into
  ``oracle/_build/<name>-<hash>/liboracle_<name>.so``.
* ``build_kats()``            the known-answer drivers against oracle/*.hpp -> ``oracle/_build/``.
* ``build_reference_kats(reference_root)``  the same drivers compiled against the reference's own
  sources where they lie (``data_struct_shared.cuh`` and the checked-in generated ``merged_spmv.h``),
  outputs only into ``oracle/_ref/``; run here to refresh ``tests/golden/*.json``.  The reference's
  two OpenMP skeletons are template text with ``${...}`` slots that need its generator (and, through
  it, the EASIER tracer that is not installed), so they are not built.
"""
from __future__ import annotations

import json
import os
import subprocess
import sys
from typing import Dict, List, Optional

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))

from flexspmv_amd.ir import FusedGraphIR  # noqa: E402
from oracle.gen_oracle import generate_oracle_source  # noqa: E402

BUILD_DIR = os.path.join(HERE, "_build")
REF_DIR = os.path.join(HERE, "_ref")
GOLDEN_DIR = os.path.join(os.path.dirname(HERE), "tests", "golden")
CXX = os.environ.get("CXX", "g++")
# x86-64-v3 (AVX2 + FMA) rather than -march=native: the libraries are built on one machine and run on another
CXXFLAGS = ["-O3", "-std=c++17", "-fopenmp", "-march=x86-64-v3", "-fPIC"]


def _run(cmd: List[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("oracle build failed:\n" + " ".join(cmd) + "\n" + proc.stdout)


def oracle_library_path(ir: FusedGraphIR) -> str:
    return os.path.join(BUILD_DIR, f"{ir.name}-{ir.content_hash()}", f"liboracle_{ir.name}.so")


def build_graph_oracle(ir: FusedGraphIR, force: bool = False) -> str:
    lib = oracle_library_path(ir)
    d = os.path.dirname(lib)
    os.makedirs(d, exist_ok=True)
    src_path = os.path.join(d, f"oracle_{ir.name}.cpp")
    src = generate_oracle_source(ir)
    old = open(src_path).read() if os.path.exists(src_path) else None
    stamp = lib + ".stamp"
    digest = str(hash_files())
    if (not force and old == src and os.path.exists(lib) and os.path.exists(stamp)
            and open(stamp).read() == digest):
        return lib
    with open(src_path, "w") as f:
        f.write(src)
    _run([CXX, *CXXFLAGS, "-shared", f"-I{HERE}", src_path, "-o", lib])
    with open(stamp, "w") as f:
        f.write(digest)
    return lib


def hash_files() -> str:
    import hashlib
    h = hashlib.sha1()
    for fn in ("tensor_ref.hpp", "merge_ref.hpp"):
        with open(os.path.join(HERE, fn), "rb") as f:
            h.update(f.read())
    h.update(" ".join(CXXFLAGS).encode())
    return h.hexdigest()


def build_kats() -> Dict[str, str]:
    os.makedirs(BUILD_DIR, exist_ok=True)
    out = {}
    for name in ("tensor_kat", "merge_kat"):
        exe = os.path.join(BUILD_DIR, name)
        _run([CXX, "-O2", "-std=c++17", "-fopenmp", f"-I{HERE}", os.path.join(HERE, name + ".cpp"), "-o", exe])
        out[name] = exe
    return out


def build_merge_capi() -> str:
    """C entry points over merge_ref.hpp for the brute-force tests -> oracle/_build/libmerge_ref.so."""
    os.makedirs(BUILD_DIR, exist_ok=True)
    lib = os.path.join(BUILD_DIR, "libmerge_ref.so")
    _run([CXX, "-O2", "-std=c++17", "-fPIC", "-shared", f"-I{HERE}", os.path.join(HERE, "merge_capi.cpp"), "-o", lib])
    return lib


def build_reference_kats(reference_root: str = "/root/reference") -> Dict[str, str]:
    os.makedirs(REF_DIR, exist_ok=True)
    out = {}
    for name in ("tensor_kat", "merge_kat"):
        exe = os.path.join(REF_DIR, name + "_ref")
        _run([CXX, "-O2", "-std=c++17", "-fopenmp", "-w", "-DKAT_REFERENCE", f"-I{reference_root}",
              os.path.join(HERE, name + ".cpp"), "-o", exe])
        out[name] = exe
    return out


def kat_lines(exe: str) -> Dict[str, str]:
    """Run a KAT driver; {"<case> <type>": "<values>"}."""
    text = subprocess.run([exe], stdout=subprocess.PIPE, check=True, text=True).stdout
    lines = {}
    for line in text.splitlines():
        parts = line.split(" ", 2)
        lines[parts[0] + " " + parts[1]] = parts[2] if len(parts) > 2 else ""
    return lines


def refresh_golden(reference_root: str = "/root/reference") -> None:
    """Rewrite tests/golden/{tensor,merge}_kat.json from the reference's own sources."""
    exes = build_reference_kats(reference_root)
    os.makedirs(GOLDEN_DIR, exist_ok=True)
    for name, exe in exes.items():
        with open(os.path.join(GOLDEN_DIR, name + ".json"), "w") as f:
            json.dump({"made_by": f"oracle/build_oracle.py refresh_golden: oracle/{name}.cpp compiled with "
                                  f"-DKAT_REFERENCE against the reference's data_struct_shared.cuh / merged_spmv.h",
                       "lines": kat_lines(exe)}, f, indent=1, sort_keys=True)


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "refresh-golden":
        refresh_golden(*(sys.argv[2:3]))
    else:
        print(build_kats())
