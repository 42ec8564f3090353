"""Generate and compile one gfx950 shared library per fused sub-graph.

The reference writes generated sources into its project root / ``include/`` and JIT-builds them with
``torch.utils.cpp_extension.load`` from a hard-coded path, copying snapshots around so that parallel
builds do not overwrite each other (test_full/easier_full.py:281-482).  Here every sub-graph gets its
own directory keyed by the content hash of its six-list description::

    flexspmv_amd/_generated/<name>-<hash>/<name>.hip
    flexspmv_amd/_generated/<name>-<hash>/lib<name>.so

so builds are independent, cacheable and parallel.  Libraries are built in-tree with ``hipcc
--offload-arch=gfx950``; a prebuilt library is used as is when its source text is unchanged.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor
from typing import Any, Dict, Iterable, List, Optional, Sequence, Tuple

from .ir import FusedGraphIR

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_ROOT = os.path.dirname(PKG_DIR)
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
INCLUDE_DIR = os.path.join(REPO_ROOT, "include")
GENERATED_DIR = os.path.join(PKG_DIR, "_generated")

OFFLOAD_ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={OFFLOAD_ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed-FP32 instructions are kept out of every kernel of this package
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


class BuildError(RuntimeError):
    pass


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise BuildError("hipcc not found: a generated FlexSpmv library cannot be built on this machine")


def _csrc_digest() -> str:
    """Digest of the headers a generated library is built from."""
    h = hashlib.sha1()
    for root in (CSRC_DIR, INCLUDE_DIR):
        for fn in sorted(os.listdir(root)):
            if fn.endswith((".hpp", ".h")) and fn != "flexspmv_formats.h":
                with open(os.path.join(root, fn), "rb") as f:
                    h.update(fn.encode())
                    h.update(f.read())
    return h.hexdigest()[:12]


def graph_dir(ir: FusedGraphIR, out_dir: Optional[str] = None) -> str:
    return os.path.join(out_dir or GENERATED_DIR, f"{ir.name}-{ir.content_hash()}")


def write_generated_source(ir: FusedGraphIR, out_dir: Optional[str] = None,
                           dtypes: Optional[Sequence[str]] = None,
                           policy: Optional[Dict[str, int]] = None,
                           defines: Sequence[str] = ()) -> Tuple[str, Dict[str, Any]]:
    """Emit ``<name>.hip`` for a sub-graph; returns (path, signature)."""
    from .codegen.merged_gen_gpu import generate_hip_source
    src, signature = generate_hip_source(ir, dtypes=dtypes, policy=policy, defines=defines)
    d = graph_dir(ir, out_dir)
    os.makedirs(d, exist_ok=True)
    path = os.path.join(d, f"{ir.name}.hip")
    old = None
    if os.path.exists(path):
        with open(path) as f:
            old = f.read()
    if old != src:
        with open(path, "w") as f:
            f.write(src)
    return path, signature


def library_path(ir: FusedGraphIR, out_dir: Optional[str] = None) -> str:
    return os.path.join(graph_dir(ir, out_dir), f"lib{ir.name}.so")


def _stamp_path(lib: str) -> str:
    return lib + ".stamp"


def _stamp(src_path: str) -> str:
    with open(src_path, "rb") as f:
        return hashlib.sha1(f.read()).hexdigest() + ":" + _csrc_digest() + ":" + " ".join(HIPCC_FLAGS)


def is_current(ir: FusedGraphIR, out_dir: Optional[str] = None) -> bool:
    lib = library_path(ir, out_dir)
    src = os.path.join(graph_dir(ir, out_dir), f"{ir.name}.hip")
    if not (os.path.exists(lib) and os.path.exists(src) and os.path.exists(_stamp_path(lib))):
        return False
    with open(_stamp_path(lib)) as f:
        return f.read() == _stamp(src)


def compile_graph(ir: FusedGraphIR, out_dir: Optional[str] = None, force: bool = False,
                  dtypes: Optional[Sequence[str]] = None, policy: Optional[Dict[str, int]] = None,
                  extra_flags: Sequence[str] = ()) -> str:
    """Generate + compile; returns the path of the shared library.  ``-DFLEX_TUNE_*`` entries of
    ``extra_flags`` are tuning switches: the generator records them in the library's signature."""
    defines = [f[2:] for f in extra_flags if f.startswith("-DFLEX_TUNE_")]
    src, _ = write_generated_source(ir, out_dir, dtypes=dtypes, policy=policy, defines=defines)
    lib = library_path(ir, out_dir)
    if not force and is_current(ir, out_dir):
        return lib
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, f"-I{CSRC_DIR}", f"-I{INCLUDE_DIR}", src, "-o", lib]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise BuildError(f"hipcc failed for sub-graph {ir.name!r}:\n{' '.join(cmd)}\n{proc.stdout}")
    with open(_stamp_path(lib), "w") as f:
        f.write(_stamp(src))
    return lib


def compile_many(graphs: Iterable[FusedGraphIR], jobs: int = 8, force: bool = False) -> List[str]:
    graphs = list(graphs)
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(graphs) or 1))) as pool:
        return list(pool.map(lambda g: compile_graph(g, force=force), graphs))


# ---------------------------------------------------------------------------------------------
# the edge-list preparation library (one per package, not per sub-graph)
# ---------------------------------------------------------------------------------------------
FORMATS_SOURCE = os.path.join(CSRC_DIR, "flex_formats.hip")
FORMATS_LIBRARY = os.path.join(GENERATED_DIR, "libflexspmv_formats.so")


def _formats_stamp() -> str:
    h = hashlib.sha1()
    for path in (FORMATS_SOURCE, os.path.join(INCLUDE_DIR, "flexspmv_formats.h")):
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest() + ":" + " ".join(HIPCC_FLAGS)


def formats_is_current() -> bool:
    stamp = _stamp_path(FORMATS_LIBRARY)
    if not (os.path.exists(FORMATS_LIBRARY) and os.path.exists(stamp)):
        return False
    with open(stamp) as f:
        return f.read() == _formats_stamp()


def compile_formats(force: bool = False) -> str:
    """Compile csrc/flex_formats.hip into _generated/libflexspmv_formats.so; returns its path."""
    if not force and formats_is_current():
        return FORMATS_LIBRARY
    os.makedirs(GENERATED_DIR, exist_ok=True)
    cmd = [hipcc_path(), *HIPCC_FLAGS, f"-I{INCLUDE_DIR}", FORMATS_SOURCE, "-o", FORMATS_LIBRARY]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise BuildError(f"hipcc failed for the formats library:\n{' '.join(cmd)}\n{proc.stdout}")
    with open(_stamp_path(FORMATS_LIBRARY), "w") as f:
        f.write(_formats_stamp())
    return FORMATS_LIBRARY


# ---------------------------------------------------------------------------------------------
# the calibration kernel of bench.py (reads and writes without arithmetic)
# ---------------------------------------------------------------------------------------------
CALIBRATE_SOURCE = os.path.join(CSRC_DIR, "flex_calibrate.hip")
CALIBRATE_LIBRARY = os.path.join(GENERATED_DIR, "libflexspmv_calibrate.so")


def compile_calibrate(force: bool = False) -> str:
    """Compile csrc/flex_calibrate.hip into _generated/libflexspmv_calibrate.so; returns its path."""
    if (not force and os.path.exists(CALIBRATE_LIBRARY)
            and os.path.getmtime(CALIBRATE_LIBRARY) >= os.path.getmtime(CALIBRATE_SOURCE)):
        return CALIBRATE_LIBRARY
    os.makedirs(GENERATED_DIR, exist_ok=True)
    cmd = [hipcc_path(), *HIPCC_FLAGS, CALIBRATE_SOURCE, "-o", CALIBRATE_LIBRARY]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise BuildError(f"hipcc failed for the calibration kernel:\n{' '.join(cmd)}\n{proc.stdout}")
    return CALIBRATE_LIBRARY


# ---------------------------------------------------------------------------------------------
# python -m flexspmv_amd.build --graph NAME [--policy BLOCKxIPT] [-D SWITCH[=VALUE]]... [--out DIR]
# ---------------------------------------------------------------------------------------------
VARIANTS_DIR = os.path.join(GENERATED_DIR, "variants")


def compile_variant(name: str, policy: Optional[str] = None, defines: Sequence[str] = (),
                    out_dir: Optional[str] = None) -> str:
    """Compile a sub-graph of flexspmv_amd.graphs with another tile shape (``"128x4"``: threads per block x
    merge items per thread) and / or tuning switches (the ``FLEX_TUNE_*`` macros of csrc/), into a
    directory of its own, for measurements next to the shipped library (``bench.py --library``)."""
    from . import graphs
    tag = "-".join([policy or "shipped", *[d.replace("=", "_") for d in defines]])
    pol = None
    if policy:
        block, ipt = (int(v) for v in policy.lower().split("x"))
        pol = {"block": block, "ipt_f32": ipt, "ipt_f64": ipt}
    return compile_graph(graphs.get(name), out_dir=os.path.join(out_dir or VARIANTS_DIR, tag), force=True, policy=pol,
                         extra_flags=[f"-D{d}" for d in defines])


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser(description="build a variant of a sub-graph library (tile shape, tuning switches)")
    ap.add_argument("--graph", required=True)
    ap.add_argument("--policy", default=None, help="BLOCKxIPT, e.g. 128x4 (default: the generator's choice)")
    ap.add_argument("-D", dest="defines", action="append", default=[], help="FLEX_TUNE_* switch, e.g. FLEX_TUNE_NT_LOADS")
    ap.add_argument("--out", default=None, help=f"directory (default {VARIANTS_DIR})")
    a = ap.parse_args()
    print(compile_variant(a.graph, a.policy, a.defines, a.out))
